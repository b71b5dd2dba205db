"""Builder for the textual form of Accelerate's fused array program.

The backend library consumes the term that the reference's optimiser hands to a
backend: a ``DelayedOpenAfun`` (``Trafo/Delayed.hs:42-59``) whose array nodes are
``PreOpenAcc`` constructors (``AST.hs:230-460``) and whose scalar code is
``OpenExp`` / ``OpenFun`` (``AST.hs:494-645``) over ``PrimFun`` (``AST.hs:661-753``).
Since that term lives in a Haskell heap, it crosses the C boundary as text: one
S-expression per constructor, de Bruijn indices kept exactly as in the reference
(``AST/Idx.hs``; index 0 is the most recently bound variable).  This module builds
such text from Python so that tests and benchmarks can state programs the way the
reference's own tests do; it contains no evaluation logic.

A program is wrapped as ``(acchip-ir 1 AFUN)``: the number is the version of this grammar
(docs/WIRE.md is its normative statement; the library refuses versions it does not know).

Grammar (atoms are bare words; every list starts with its constructor name):

  scalar type   i8 i16 i32 i64 u8 u16 u32 u64 f16 f32 f64   (Int = i64, Word = u64,
                PrimBool / TAG = u8, ``Type.hs:112-152``) | v<N><SCALAR> for the SIMD
                vector `Vec N t`, N in 2 3 4 8 16 (one leaf, components side by side)
  tuple type    unit | SCALAR | (pair T T)
  array type    (array RANK T)          arrays type  unit | ARRAY | (pair AS AS)
  lhs           (single T) | (wild T) | (pair LHS LHS)        (``AST/LeftHandSide.hs``)

  exp  (let LHS e e) (var I) (pair e e) nil (const SCALAR lit) (undef SCALAR)
       (minbound T) (maxbound T) (pi T) (prim NAME T.. e) (toindex RANK sh ix)
       (fromindex RANK sh i) (indexslice SLICE slix sh) (indexfull SLICE slix sl)
       (case e ((TAG e)..) DEFAULT|none) (cond e e e) (while FUN FUN e)
       (index A ix) (linearindex A i) (shape A) (shapesize RANK sh)
       (coerce T T e) (foreign FUN e) (vecpack N SCALAR e) (vecunpack N SCALAR e)
  fun  (lam LHS fun) | exp
  acc  (avar I) (alet ALHS acc acc) (apair acc acc) anil (apply AFUN acc)
       (acond exp acc acc) (awhile AFUN AFUN acc) (use ARRAY SLOT) (unit T exp)
       (reshape RANK sh acc) (generate ARRAY sh fun) (transform ARRAY sh fun fun acc)
       (replicate SLICE slix acc) (slice SLICE acc slix) (map T fun acc)
       (zipwith T fun acc acc) (fold fun (just e)|nothing acc)
       (foldseg ITYPE fun (just e)|nothing acc acc) (scan l|r fun (just e)|nothing acc)
       (scan' l|r fun e acc) (permute fun acc fun acc) (backpermute RANK sh fun acc)
       (stencil STENCIL T fun BOUNDARY acc) (stencil2 STENCIL STENCIL T fun B acc B acc)
       (delayed ARRAY extent indexD linearIndexD)      -- a fused operand
  afun (alam ALHS afun) | acc
"""
from __future__ import annotations

import math
import struct
import threading

WIRE_VERSION = 1   # of the grammar above; the library refuses any other

# --------------------------------------------------------------------------------------
# types

SCALARS = ("i8", "i16", "i32", "i64", "u8", "u16", "u32", "u64", "f16", "f32", "f64")
i8, i16, i32, i64, u8, u16, u32, u64, f16, f32, f64 = SCALARS
Int = i64
Word = u64
Bool = u8
unit = "unit"

INTEGRAL = ("i8", "i16", "i32", "i64", "u8", "u16", "u32", "u64")
FLOATING = ("f16", "f32", "f64")


def tvec(n, t):
    """SIMD vector type `Vec n t` (n in 2, 3, 4, 8, 16), one scalar leaf written v<n><t>."""
    assert n in (2, 3, 4, 8, 16) and t in SCALARS
    return "v%d%s" % (n, t)


def vec_of(t):
    """'v3i32' -> (3, 'i32'), anything else -> None."""
    if isinstance(t, str) and t[0] == "v":
        k = 1
        while k < len(t) and t[k].isdigit():
            k += 1
        if 1 < k < len(t) and t[k:] in SCALARS:
            return int(t[1:k]), t[k:]
    return None


def tpair(a, b):
    return ("pair", a, b)


def ttup(*ts):
    """Representation type of a surface tuple: (((), a), b) .. (Sugar/Elt.hs:81-131)."""
    t = unit
    for x in ts:
        t = tpair(t, x)
    return t


def tshape(rank):
    """Representation type of a shape of the given rank (Representation/Shape.hs:31-46)."""
    return ttup(*([Int] * rank))


def tarray(rank, t):
    return ("array", rank, t)


def tleaves(t):
    if t == unit:
        return []
    if isinstance(t, str):
        return [t]
    assert t[0] == "pair", t
    return tleaves(t[1]) + tleaves(t[2])


# --------------------------------------------------------------------------------------
# rendering

def _atom(x):
    if isinstance(x, bool):
        return "1" if x else "0"
    if isinstance(x, int):
        return str(x)
    if isinstance(x, float):
        if math.isnan(x):
            return "nan"
        if math.isinf(x):
            return "inf" if x > 0 else "-inf"
        return x.hex()
    return str(x)


def render(x):
    if isinstance(x, (tuple, list)):
        return "(" + " ".join(render(y) for y in x) + ")"
    return _atom(x)


class _Scope(threading.local):
    def __init__(self):
        self.d = 0   # scalar variables in scope
        self.ad = 0  # array variables in scope


_scope = _Scope()


class Node:
    """A term under construction.  ``sx(d, ad)`` renders it with ``d`` scalar and ``ad``
    array variables in scope, turning binder levels into de Bruijn indices."""

    def sx(self, d, ad):
        raise NotImplementedError

    def text(self):
        """The program as it crosses the C boundary: (acchip-ir VERSION term)."""
        return "(acchip-ir %d %s)" % (WIRE_VERSION, render(self.sx(0, 0)))


class Raw(Node):
    def __init__(self, head, *args):
        self.head = head
        self.args = args

    def sx(self, d, ad):
        out = [self.head]
        for a in self.args:
            out.append(_sx(a, d, ad))
        return tuple(out) if self.args or not isinstance(self.head, str) else self.head


def _sx(a, d, ad):
    if isinstance(a, Node):
        return a.sx(d, ad)
    if isinstance(a, (tuple, list)) and any(isinstance(y, (Node, tuple, list)) for y in a):
        return tuple(_sx(y, d, ad) for y in a)
    return a


class Var(Node):
    def __init__(self, level, ty):
        self.level = level
        self.ty = ty

    def sx(self, d, ad):
        ix = d - 1 - self.level
        assert ix >= 0, "scalar variable used outside its scope"
        return ("var", ix)


class AVar(Node):
    def __init__(self, level, ty):
        self.level = level
        self.ty = ty

    def sx(self, d, ad):
        ix = ad - 1 - self.level
        assert ix >= 0, "array variable used outside its scope"
        return ("avar", ix)


class _AIdx(Node):
    """Bare de Bruijn index of an array variable, for Index / LinearIndex / Shape."""

    def __init__(self, av):
        assert isinstance(av, AVar), "array operand of a scalar term must be a variable"
        self.av = av

    def sx(self, d, ad):
        return ad - 1 - self.av.level


class wild:
    """Marks a component of a left-hand side that binds nothing (LeftHandSideWildcard)."""

    def __init__(self, ty):
        self.ty = ty


def _lhs(ty, level, mk):
    """Returns (lhs sexpr, value tree of variables, number bound)."""
    if isinstance(ty, wild):
        return ("wild", ty.ty), None, 0
    if ty == unit:
        return ("wild", unit), None, 0
    if isinstance(ty, str) or ty[0] == "array":
        return ("single", ty), mk(level, ty), 1
    assert ty[0] == "pair"
    l1, v1, n1 = _lhs(ty[1], level, mk)
    l2, v2, n2 = _lhs(ty[2], level + n1, mk)
    return ("pair", l1, l2), (v1, v2), n1 + n2


class _Bind(Node):
    """(head pre.. LHS scoped..): binds the variables of ``ty`` in each scoped term."""

    def __init__(self, head, ty, pre, scoped_fns, array=False):
        self.head, self.pre, self.array = head, pre, array
        if array:
            self.lhs, vars_, self.n = _lhs(ty, _scope.ad, AVar)
            _scope.ad += self.n
        else:
            self.lhs, vars_, self.n = _lhs(ty, _scope.d, Var)
            _scope.d += self.n
        try:
            self.scoped = [f(vars_) for f in scoped_fns]
        finally:
            if array:
                _scope.ad -= self.n
            else:
                _scope.d -= self.n

    def sx(self, d, ad):
        out = [self.head]
        out += [_sx(p, d, ad) for p in self.pre]
        out.append(self.lhs)
        d2, ad2 = (d, ad + self.n) if self.array else (d + self.n, ad)
        out += [_sx(s, d2, ad2) for s in self.scoped]
        return tuple(out)


def _untup(v):
    """Value tree (((None, a), b), c) of a surface tuple -> [a, b, c]."""
    out = []
    while v is not None:
        v, x = v
        out.append(x)
    return out[::-1]


# --------------------------------------------------------------------------------------
# scalar expressions (AST.hs:524-645)

def lam(tys, fn):
    """Scalar function of len(tys) arguments; fn receives one value tree per argument.
    A value tree mirrors the argument type: Var for a scalar, (l, r) for a pair, None for
    unit or wildcards."""
    tys = list(tys)

    def go(k, got):
        if k == len(tys):
            return fn(*got)
        return _Bind("lam", tys[k], [], [lambda v: go(k + 1, got + [v])])

    return go(0, [])


class _Let(Node):
    def __init__(self, ty, bound, fn):
        self.bound = bound
        self.bind = _Bind("let*", ty, [], [fn])

    def sx(self, d, ad):
        b = self.bind.sx(d, ad)  # ("let*", lhs, body)
        return ("let", b[1], _sx(self.bound, d, ad), b[2])


def let(ty, bound, fn):
    """Let lhs bound body; fn receives the value tree of the variables lhs binds."""
    return _Let(ty, bound, fn)


def pair(a, b):
    return Raw("pair", a, b)


nil = Raw("nil")


def tup(*xs):
    """Surface tuple / shape value: Pair (Pair Nil a) b."""
    e = nil
    for x in xs:
        e = pair(e, x)
    return e


def untup(v):
    return _untup(v)


def const(ty, v):
    if ty in FLOATING:
        v = float(v)
        if ty == f32 and math.isfinite(v):
            v = struct.unpack("f", struct.pack("f", v))[0]
    else:
        v = int(v)
    return Raw("const", ty, v)


def constI(v):
    return const(Int, v)


def sh(*dims):
    """Shape / index expression Z :. d0 :. d1 .. from ints or expressions."""
    return tup(*[constI(x) if isinstance(x, int) else x for x in dims])


def undef(ty):
    return Raw("undef", ty)


def minbound(ty):
    return Raw("minbound", ty)


def maxbound(ty):
    return Raw("maxbound", ty)


def pi(ty):
    return Raw("pi", ty)


def prim(name, tys, arg):
    if isinstance(tys, str):
        tys = [tys]
    return Raw("prim", name, *tys, arg)


def _bin(name):
    return lambda ty, a, b: prim(name, ty, pair(a, b))


def _un(name):
    return lambda ty, a: prim(name, ty, a)


add, sub, mul = _bin("add"), _bin("sub"), _bin("mul")
neg, abs_, sig = _un("neg"), _un("abs"), _un("sig")
quot, rem, idiv, mod = _bin("quot"), _bin("rem"), _bin("idiv"), _bin("mod")
quotrem, divmod_ = _bin("quotrem"), _bin("divmod")
band, bor, bxor, bnot = _bin("band"), _bin("bor"), _bin("bxor"), _un("bnot")
shl, shr, rotl, rotr = _bin("shl"), _bin("shr"), _bin("rotl"), _bin("rotr")
popcount, clz, ctz = _un("popcount"), _un("clz"), _un("ctz")
fdiv, recip = _bin("fdiv"), _un("recip")
sin, cos, tan, asin, acos, atan = (_un(n) for n in ("sin", "cos", "tan", "asin", "acos", "atan"))
sinh, cosh, tanh, asinh, acosh, atanh = (_un(n) for n in ("sinh", "cosh", "tanh", "asinh", "acosh", "atanh"))
exp, sqrt, log = _un("exp"), _un("sqrt"), _un("log")
fpow, logbase, atan2 = _bin("fpow"), _bin("logbase"), _bin("atan2")
isnan, isinf = _un("isnan"), _un("isinf")
lt, gt, lte, gte, eq, neq = (_bin(n) for n in ("lt", "gt", "lte", "gte", "eq", "neq"))
max_, min_ = _bin("max"), _bin("min")


def land(a, b):
    return Raw("prim", "land", pair(a, b))


def lor(a, b):
    return Raw("prim", "lor", pair(a, b))


def lnot(a):
    return Raw("prim", "lnot", a)


def truncate(ta, tb, a):
    return prim("truncate", [ta, tb], a)


def round_(ta, tb, a):
    return prim("round", [ta, tb], a)


def floor(ta, tb, a):
    return prim("floor", [ta, tb], a)


def ceiling(ta, tb, a):
    return prim("ceiling", [ta, tb], a)


def fromintegral(ta, tb, a):
    return prim("fromintegral", [ta, tb], a)


def tofloating(ta, tb, a):
    return prim("tofloating", [ta, tb], a)


def toindex(rank, sh_, ix):
    return Raw("toindex", rank, sh_, ix)


def fromindex(rank, sh_, i):
    return Raw("fromindex", rank, sh_, i)


def indexslice(spec, slix, sh_):
    return Raw("indexslice", tuple(spec), slix, sh_)


def indexfull(spec, slix, sl):
    return Raw("indexfull", tuple(spec), slix, sl)


def case(e, alts, default=None):
    return Raw("case", e, tuple((t, x) for t, x in alts), default if default is not None else "none")


def cond(c, t, e):
    return Raw("cond", c, t, e)


def while_(ty, cond_fn, body_fn, seed):
    return Raw("while", lam([ty], cond_fn), lam([ty], body_fn), seed)


def index(av, ix):
    return Raw("index", _AIdx(av), ix)


def linearindex(av, i):
    return Raw("linearindex", _AIdx(av), i)


def shape(av):
    return Raw("shape", _AIdx(av))


def untup_shape(av):
    """Extents of an array variable as a list of expressions, outermost first."""
    rank = int(av.ty[1])
    sht = tshape(rank)
    return [let(sht, shape(av), (lambda k: lambda s: _untup(s)[k])(k)) for k in range(rank)]


def shapesize(rank, sh_):
    return Raw("shapesize", rank, sh_)


def vecpack(n, t, e):
    """VecPack: a tuple of n components of type t -> Vec n t  (Interpreter.hs:942)."""
    return Raw("vecpack", n, t, e)


def vecunpack(n, t, e):
    """VecUnpack: Vec n t -> the tuple of its components  (Interpreter.hs:943)."""
    return Raw("vecunpack", n, t, e)


def coerce(t1, t2, e):
    return Raw("coerce", t1, t2, e)


def foreign(fun, e):
    return Raw("foreign", fun, e)


def just(ix):
    """PrimMaybe value Just ix = (1, ((), ix))  (AST.hs:202)."""
    return pair(const(u8, 1), pair(nil, ix))


def nothing(ty):
    """PrimMaybe value Nothing = (0, ((), undef..)) for an index of type ty."""
    def und(t):
        if t == unit:
            return nil
        if isinstance(t, str):
            return undef(t)
        return pair(und(t[1]), und(t[2]))
    return pair(const(u8, 0), pair(nil, und(ty)))


# --------------------------------------------------------------------------------------
# array terms (AST.hs:230-460)

def alam(tys, fn):
    """Array function: tys are array types (or tuples of them); the first argument is
    bound first, so the last one has de Bruijn index 0 (Interpreter.hs:124)."""
    tys = list(tys)

    def go(k, got):
        if k == len(tys):
            return fn(*got)
        return _Bind("alam", tys[k], [], [lambda v: go(k + 1, got + [v])], array=True)

    return go(0, [])


class _ALet(Node):
    def __init__(self, ty, bound, fn):
        self.bound = bound
        self.bind = _Bind("alet*", ty, [], [fn], array=True)

    def sx(self, d, ad):
        b = self.bind.sx(d, ad)
        return ("alet", b[1], _sx(self.bound, d, ad), b[2])


def alet(ty, bound, fn):
    return _ALet(ty, bound, fn)


def apair(a, b):
    return Raw("apair", a, b)


anil = Raw("anil")


def apply(afun, acc):
    return Raw("apply", afun, acc)


def _hex(text):
    return text.encode().hex() or "-"


def atrace(msg, traced, body):
    """Atrace msg traced body (AST.hs Atrace; evaluated as Interpreter.hs:215)."""
    return Raw("atrace", _hex(msg), traced, body)


class _Closed(Node):
    """A closed term (built outside every binder): rendered in an empty environment."""

    def __init__(self, term):
        self.term = term

    def sx(self, d, ad):
        return self.term.sx(0, 0)


def aforeign(name, afun, acc):
    """Aforeign with its pure fallback afun, a closed array function built outside every
    binder (Interpreter.hs:217 evaluates it in the empty environment)."""
    return Raw("aforeign", _hex(name), _Closed(afun), acc)


def acond(e, a1, a2):
    return Raw("acond", e, a1, a2)


def awhile(ty, cond_fn, body_fn, acc):
    return Raw("awhile", alam([ty], cond_fn), alam([ty], body_fn), acc)


def use(aty, slot):
    return Raw("use", aty, slot)


def unit_(ty, e):
    return Raw("unit", ty, e)


def reshape(rank, sh_, acc):
    return Raw("reshape", rank, sh_, acc)


def generate(aty, sh_, fun):
    return Raw("generate", aty, sh_, fun)


def transform(aty, sh_, p, f, acc):
    return Raw("transform", aty, sh_, p, f, acc)


def replicate(spec, slix, acc):
    return Raw("replicate", tuple(spec), slix, acc)


def slice_(spec, acc, slix):
    return Raw("slice", tuple(spec), acc, slix)


def map_(ty, fun, acc):
    return Raw("map", ty, fun, acc)


def zipwith(ty, fun, a1, a2):
    return Raw("zipwith", ty, fun, a1, a2)


def _seed(z):
    return "nothing" if z is None else Raw("just", z)


def fold(fun, z, acc):
    return Raw("fold", fun, _seed(z), acc)


def foldseg(ity, fun, z, acc, seg):
    return Raw("foldseg", ity, fun, _seed(z), acc, seg)


def scan(direction, fun, z, acc):
    return Raw("scan", direction, fun, _seed(z), acc)


def scan_(direction, fun, z, acc):
    return Raw("scan'", direction, fun, z, acc)


def permute(fun, defaults, p, acc):
    return Raw("permute", fun, defaults, p, acc)


def backpermute(rank, sh_, p, acc):
    return Raw("backpermute", rank, sh_, p, acc)


def stencil(sr, ty, fun, boundary, acc):
    return Raw("stencil", sr, ty, fun, boundary, acc)


def stencil2(sr1, sr2, ty, fun, b1, a1, b2, a2):
    return Raw("stencil2", sr1, sr2, ty, fun, b1, a1, b2, a2)


def delayed(aty, extent, index_fn, linear_fn):
    return Raw("delayed", aty, extent, index_fn, linear_fn)


# stencil shapes (Representation/Stencil.hs:34-60)
def sunit(n, ty):
    return ("unit%d" % n, ty)


def stup(*subs):
    return ("tup%d" % len(subs),) + tuple(subs)


def stencil_type(sr):
    """Representation type of the stencil function's argument."""
    if sr[0].startswith("unit"):
        return ttup(*([sr[1]] * int(sr[0][4:])))
    return ttup(*[stencil_type(s) for s in sr[1:]])


clamp, mirror, wrap = "clamp", "mirror", "wrap"


def constant(ty, value_tree):
    """Constant boundary; value_tree mirrors ty with Python numbers at the leaves."""
    def go(t, v):
        if t == unit:
            return nil
        if isinstance(t, str):
            return const(t, v)
        return pair(go(t[1], v[0]), go(t[2], v[1]))
    return Raw("constant", go(ty, value_tree))


def function(fun):
    return Raw("function", fun)


# --------------------------------------------------------------------------------------
# what Trafo.Fusion hands over for common surface idioms (Trafo/Fusion.hs:139-216)

def delayed_var(av):
    """A consumer's operand that is a plain variable arrives as Manifest (Avar v)."""
    return av


def delayed_zipwith(ty_out, rank, f, a1, t1, a0, t0):
    """zipWith f a1 a0 over two distinct manifest variables: the Yield form with
    extent = intersect (shape a1) (shape a0), indexD = \\ix -> f (a1!ix) (a0!ix) and
    linearIndexD = indexD . fromIndex extent (Trafo/Fusion.hs:149,1205-1233,1689-1714)."""
    sht = tshape(rank)

    def extent():
        def comp(s1, s0):
            l1, l0 = _untup(s1), _untup(s0)
            return tup(*[min_(Int, x, y) for x, y in zip(l1, l0)])
        return let(sht, shape(a1), lambda s1: let(sht, shape(a0), lambda s0: comp(s1, s0)))

    def body(ix):
        return let(t1, index(a1, ix), lambda x: let(t0, index(a0, ix), lambda y: f(x, y)))

    def vt(v):  # value tree -> expression
        if v is None:
            return nil
        if isinstance(v, tuple):
            return pair(vt(v[0]), vt(v[1]))
        return v

    index_fn = lam([sht], lambda ix: body(vt(ix)))
    linear_fn = lam([Int], lambda i: let(sht, fromindex(rank, extent(), i), lambda ix: body(vt(ix))))
    return delayed(tarray(rank, ty_out), extent(), index_fn, linear_fn)


def vexp(v):
    """Value tree of variables -> expression rebuilding the same value."""
    if v is None:
        return nil
    if isinstance(v, tuple):
        return pair(vexp(v[0]), vexp(v[1]))
    return v

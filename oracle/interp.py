"""ORACLE -- test infrastructure, not product code.

A sequential CPU restatement of the reference interpreter, evaluating the same textual
program the HIP backend consumes.  Only tests/, __graft_entry__.smoke() and the
cpu_baseline leg of bench.py may import this module.  It is written for fidelity to
the reference's traversal order and arithmetic, not speed: use it on small inputs.

What it follows (paths relative to the reference's src/Data/Array/Accelerate):
  run / runN / evalOpenAfun / evalOpenAcc     Interpreter.hs:93-126, 168-259
  producers (unit, generate, transform, ...)  Interpreter.hs:265-368, 627-634
  fold / fold1 / foldSeg / fold1Seg           Interpreter.hs:371-424, Shape.hs:127-142
  scanl scanl1 scanl' scanr scanr1 scanr'     Interpreter.hs:427-582
  permute                                     Interpreter.hs:585-624
  stencil, stencil2, stencilAccess, bounded   Interpreter.hs:637-839
  scalar evaluator and primitive tables       Interpreter.hs:888-1416
  size / toIndex / fromIndex / intersect      Representation/Shape.hs:67-120
  fromFunction traversal (row-major)          Representation/Array.hs:102-122

Pinned by tests/test_oracle_golden.py against the reference's own doctest outputs and
issue regression vectors (tests/golden/*.json) and against closed forms, and by
tests/test_oracle_pins.py for what those vectors leave open: every scalar primitive on every
type against Python's unbounded integers, numpy and struct; stencils of ranks 1-4 and stencil2
by brute force; fold1Seg against foldl1 over split places; transform; SIMD pack / unpack; and by
tests/test_oracle_control_pins.py for the array-level control flow (alet, apair, apply, aforeign,
acond, awhile, atrace, use, unit, reshape: every program the GPU suite runs through these branches
against the same computation in numpy, plus while-before-step, closed fallbacks, slot numbers and
de Bruijn levels).  No branch of eval_acc that a GPU test reaches is without such a pin.
Parity unpinned: the last-ulp behaviour of transcendental primitives (libm here, GHC's in the
reference), and the exact shapes of the terms the reference's fusion emits.

Value representation: unit is (), pairs are 2-tuples, shapes are nested pairs
(((), d_outer), d_inner) exactly as in the reference.  Integers are Python ints
wrapped to their width after every operation (Haskell fixed-width semantics);
f64 is a Python float; f32 / f16 are numpy scalars so every operation rounds once.
"""
from __future__ import annotations

import math

import numpy as np

INT_BITS = {"i8": 8, "i16": 16, "i32": 32, "i64": 64, "u8": 8, "u16": 16, "u32": 32, "u64": 64}
NP = {"i8": np.int8, "i16": np.int16, "i32": np.int32, "i64": np.int64,
      "u8": np.uint8, "u16": np.uint16, "u32": np.uint32, "u64": np.uint64,
      "f16": np.float16, "f32": np.float32, "f64": np.float64}
FLOATS = ("f16", "f32", "f64")


def vec_of(ty):
    """'v3i32' -> (3, 'i32') for a SIMD vector type `Vec n t`, else None.  A vector value is a
    Python tuple of its components; its buffer holds them side by side (Array/Data.hs:119,190)."""
    if isinstance(ty, str) and ty[0] == "v":
        k = 1
        while k < len(ty) and ty[k].isdigit():
            k += 1
        if 1 < k < len(ty) and ty[k:] in NP and int(ty[1:k]) in (2, 3, 4, 8, 16):
            return int(ty[1:k]), ty[k:]
    return None


def _scalar_out(ty, v):
    if ty in INT_BITS:
        return int(v)
    return float(v) if ty == "f64" else v


class OracleError(Exception):
    """A condition the reference reports through boundsCheck / internalError."""


# --------------------------------------------------------------------------------------
# reader

TRACE = []   # (message, traced arrays) of every Atrace node evaluated, in order


def parse(text):
    toks = text.replace("(", " ( ").replace(")", " ) ").split()
    pos = 0

    def rd():
        nonlocal pos
        t = toks[pos]
        pos += 1
        if t == "(":
            out = []
            while toks[pos] != ")":
                out.append(rd())
            pos += 1
            return out
        return t

    x = rd()
    assert pos == len(toks), "trailing input"
    # a program travels as (acchip-ir VERSION afun); scalar and array terms inside tests come bare
    if isinstance(x, list) and x and x[0] == "acchip-ir":
        if x[1] != "1":
            raise OracleError("unsupported wire format version " + str(x[1]))
        x = x[2]
    return x


# --------------------------------------------------------------------------------------
# scalars

def wrap(ty, x):
    b = INT_BITS[ty]
    x &= (1 << b) - 1
    if ty[0] == "i" and x >> (b - 1):
        x -= 1 << b
    return x


def fl(ty, x):
    if ty == "f64":
        return float(x)
    return NP[ty](x)


def literal(ty, tok):
    if ty in FLOATS:
        if tok in ("nan", "inf", "-inf"):
            return fl(ty, float(tok))
        return fl(ty, float.fromhex(tok) if "x" in tok else float(tok))
    return wrap(ty, int(tok, 0))


def from_bool(b):
    return 1 if b else 0


def _quot(a, b):
    if b == 0:
        raise OracleError("divide by zero")
    q = abs(a) // abs(b)
    return -q if (a < 0) != (b < 0) else q


def _unsigned(ty, x):
    return x & ((1 << INT_BITS[ty]) - 1)


def _shl(ty, a, n):
    return 0 if n >= INT_BITS[ty] else wrap(ty, a << n)


def _shr(ty, a, n):
    if n >= INT_BITS[ty]:
        return -1 if a < 0 else 0
    return a >> n  # arithmetic on negative Python ints, logical on unsigned values


def _rotl(ty, a, n):
    b = INT_BITS[ty]
    n %= b
    u = _unsigned(ty, a)
    return wrap(ty, (u << n) | (u >> (b - n))) if n else a


def _clz(ty, a):
    b = INT_BITS[ty]
    return b - _unsigned(ty, a).bit_length()


def _ctz(ty, a):
    u = _unsigned(ty, a)
    return INT_BITS[ty] if u == 0 else (u & -u).bit_length() - 1


def _signum_f(ty, x):
    # GHC.Float: signum x | x > 0 = 1 | x < 0 = -1 | otherwise = x
    return fl(ty, 1) if x > 0 else fl(ty, -1) if x < 0 else x


def _fmath(name):
    f = getattr(np, name)

    def go(ty, x):
        with np.errstate(all="ignore"):
            return fl(ty, f(NP[ty](x)))
    return go


def _round_half_even(x):
    x = float(x)
    if math.isnan(x) or math.isinf(x):
        raise OracleError("round of non-finite value")
    return round(x)


def _to_float(ty_to, ty_from, x):
    if ty_from in INT_BITS:
        return fl(ty_to, NP[ty_to](NP[ty_from](x)))  # one rounding, nearest-even
    return fl(ty_to, x)


def _hs_max(x, y):  # Ord default: max x y = if x <= y then y else x  (Interpreter.hs:1410-1412)
    return y if x <= y else x


def _hs_min(x, y):  # min x y = if x <= y then x else y  (Interpreter.hs:1414-1416)
    return x if x <= y else y


def _arith(int_op, flt_op):
    def go(ty, a, b):
        if ty in INT_BITS:
            return wrap(ty, int_op(a, b))
        with np.errstate(all="ignore"):
            return fl(ty, flt_op(a, b))
    return go


def _fdiv(ty, a, b):
    with np.errstate(all="ignore"):
        if ty == "f64":
            return float(np.float64(a) / np.float64(b))
        return a / b


def _abs(ty, a):
    return wrap(ty, abs(a)) if ty in INT_BITS else fl(ty, abs(a))


def _neg(ty, a):
    return wrap(ty, -a) if ty in INT_BITS else fl(ty, -a)


def _sig(ty, a):
    if ty in INT_BITS:
        return (a > 0) - (a < 0)
    return _signum_f(ty, a)


def _fpow(ty, a, b):
    with np.errstate(all="ignore"):
        return fl(ty, np.power(NP[ty](a), NP[ty](b)))


def _logbase(ty, a, b):  # logBase x y = log y / log x
    with np.errstate(all="ignore"):
        return fl(ty, np.log(NP[ty](b)) / np.log(NP[ty](a)))


def _atan2(ty, a, b):
    with np.errstate(all="ignore"):
        return fl(ty, np.arctan2(NP[ty](a), NP[ty](b)))


# name -> (number of leading type parameters, function(types.., argument value))
# argument values of binary primitives are pairs (Interpreter.hs:1086-1148).
PRIMS = {
    "add": (1, lambda t, v: _arith(lambda a, b: a + b, lambda a, b: a + b)(t, *v)),
    "sub": (1, lambda t, v: _arith(lambda a, b: a - b, lambda a, b: a - b)(t, *v)),
    "mul": (1, lambda t, v: _arith(lambda a, b: a * b, lambda a, b: a * b)(t, *v)),
    "neg": (1, _neg), "abs": (1, _abs), "sig": (1, _sig),
    "quot": (1, lambda t, v: wrap(t, _quot(*v))),
    "rem": (1, lambda t, v: wrap(t, v[0] - _quot(*v) * v[1])),
    "quotrem": (1, lambda t, v: (wrap(t, _quot(*v)), wrap(t, v[0] - _quot(*v) * v[1]))),
    "idiv": (1, lambda t, v: wrap(t, _idiv(*v))),
    "mod": (1, lambda t, v: wrap(t, v[0] - _idiv(*v) * v[1])),
    "divmod": (1, lambda t, v: (wrap(t, _idiv(*v)), wrap(t, v[0] - _idiv(*v) * v[1]))),
    "band": (1, lambda t, v: wrap(t, v[0] & v[1])),
    "bor": (1, lambda t, v: wrap(t, v[0] | v[1])),
    "bxor": (1, lambda t, v: wrap(t, v[0] ^ v[1])),
    "bnot": (1, lambda t, a: wrap(t, ~a)),
    "shl": (1, lambda t, v: _shl(t, *v)),
    "shr": (1, lambda t, v: _shr(t, *v)),
    "rotl": (1, lambda t, v: _rotl(t, *v)),
    "rotr": (1, lambda t, v: _rotl(t, v[0], -v[1])),
    "popcount": (1, lambda t, a: bin(_unsigned(t, a)).count("1")),
    "clz": (1, _clz), "ctz": (1, _ctz),
    "fdiv": (1, lambda t, v: _fdiv(t, *v)),
    "recip": (1, lambda t, a: _fdiv(t, fl(t, 1), a)),
    "sin": (1, _fmath("sin")), "cos": (1, _fmath("cos")), "tan": (1, _fmath("tan")),
    "asin": (1, _fmath("arcsin")), "acos": (1, _fmath("arccos")), "atan": (1, _fmath("arctan")),
    "sinh": (1, _fmath("sinh")), "cosh": (1, _fmath("cosh")), "tanh": (1, _fmath("tanh")),
    "asinh": (1, _fmath("arcsinh")), "acosh": (1, _fmath("arccosh")), "atanh": (1, _fmath("arctanh")),
    "exp": (1, _fmath("exp")), "sqrt": (1, _fmath("sqrt")), "log": (1, _fmath("log")),
    "fpow": (1, lambda t, v: _fpow(t, *v)),
    "logbase": (1, lambda t, v: _logbase(t, *v)),
    "atan2": (1, lambda t, v: _atan2(t, *v)),
    "truncate": (2, lambda ta, tb, a: wrap(tb, math.trunc(float(a)))),
    "round": (2, lambda ta, tb, a: wrap(tb, _round_half_even(a))),
    "floor": (2, lambda ta, tb, a: wrap(tb, math.floor(float(a)))),
    "ceiling": (2, lambda ta, tb, a: wrap(tb, math.ceil(float(a)))),
    "isnan": (1, lambda t, a: from_bool(math.isnan(float(a)))),
    "isinf": (1, lambda t, a: from_bool(math.isinf(float(a)))),
    "lt": (1, lambda t, v: from_bool(v[0] < v[1])),
    "gt": (1, lambda t, v: from_bool(v[0] > v[1])),
    "lte": (1, lambda t, v: from_bool(v[0] <= v[1])),
    "gte": (1, lambda t, v: from_bool(v[0] >= v[1])),
    "eq": (1, lambda t, v: from_bool(v[0] == v[1])),
    "neq": (1, lambda t, v: from_bool(v[0] != v[1])),
    "max": (1, lambda t, v: _hs_max(*v)),
    "min": (1, lambda t, v: _hs_min(*v)),
    "land": (0, lambda v: from_bool(v[0] != 0 and v[1] != 0)),   # strict in both (AST.hs:737-749)
    "lor": (0, lambda v: from_bool(v[0] != 0 or v[1] != 0)),
    "lnot": (0, lambda a: from_bool(a == 0)),
    "fromintegral": (2, lambda ta, tb, a: wrap(tb, a) if tb in INT_BITS else _to_float(tb, ta, a)),
    "tofloating": (2, lambda ta, tb, a: _to_float(tb, ta, a)),
}


def _idiv(a, b):
    if b == 0:
        raise OracleError("divide by zero")
    return a // b  # floor, as Haskell div


# --------------------------------------------------------------------------------------
# shapes (Representation/Shape.hs:67-120)

def sh_list(sh):
    out = []
    while sh != ():
        sh, d = sh
        out.append(d)
    return out[::-1]


def sh_of(dims):
    sh = ()
    for d in dims:
        sh = (sh, d)
    return sh


def size(sh):
    n = 1
    for d in sh_list(sh):
        if d <= 0:
            return 0
        n *= d
    return n


def to_index(sh, ix):
    if sh == ():
        return 0
    (sh1, sz), (ix1, i) = sh, ix
    if not (0 <= i < sz):
        raise OracleError("index out of bounds")
    return to_index(sh1, ix1) * sz + i


def from_index(sh, i):
    if sh == ():
        return ()
    sh1, sz = sh
    if sh1 == ():
        if not (0 <= i < sz):
            raise OracleError("index out of bounds")
        return ((), i)
    if sz == 0:
        raise OracleError("divide by zero")
    return (from_index(sh1, _quot(i, sz)), i - _quot(i, sz) * sz)


def intersect(a, b):
    return sh_of([min(x, y) for x, y in zip(sh_list(a), sh_list(b))])


# --------------------------------------------------------------------------------------
# arrays: struct-of-arrays payload, one flat numpy buffer per scalar leaf (Array/Data.hs:95-119)

def leaves(ty):
    if ty == "unit":
        return []
    if isinstance(ty, str):
        return [ty]
    return leaves(ty[1]) + leaves(ty[2])


class Arr:
    def __init__(self, sh, ty, bufs=None):
        self.sh, self.ty = sh, ty
        n = size(sh)
        self.bufs = bufs if bufs is not None else [
            np.zeros((n, vec_of(t)[0]), NP[vec_of(t)[1]]) if vec_of(t) else np.zeros(n, NP[t]) for t in leaves(ty)]

    def read(self, i):
        it = iter(self.bufs)

        def go(ty):
            if ty == "unit":
                return ()
            if isinstance(ty, str):
                v = next(it)[i]
                if vec_of(ty):
                    return tuple(_scalar_out(vec_of(ty)[1], x) for x in v)
                return _scalar_out(ty, v)
            a = go(ty[1])
            return (a, go(ty[2]))
        return go(self.ty)

    def write(self, i, v):
        it = iter(self.bufs)

        def go(ty, v):
            if ty == "unit":
                return
            if isinstance(ty, str):
                next(it)[i] = v
                return
            go(ty[1], v[0])
            go(ty[2], v[1])
        go(self.ty, v)

    def index(self, ix):
        return self.read(to_index(self.sh, ix))


def from_function(sh, ty, f):
    """Representation/Array.hs:102-122: fill in row-major order."""
    out = Arr(sh, ty)
    for i, ix in enumerate(indices(sh)):
        out.write(i, f(ix))
    return out


def indices(sh):
    dims = sh_list(sh)
    if any(d <= 0 for d in dims):
        return
    ix = [0] * len(dims)
    while True:
        yield sh_of(ix)
        k = len(dims) - 1
        while k >= 0:
            ix[k] += 1
            if ix[k] < dims[k]:
                break
            ix[k] = 0
            k -= 1
        if k < 0:
            return


class Delayed:
    def __init__(self, ty, sh, ixf, linf):
        self.ty, self.sh, self.ixf, self.linf = ty, sh, ixf, linf


# --------------------------------------------------------------------------------------
# environments

def push(env, lhs, v):
    k = lhs[0]
    if k == "single":
        return env + (v,)
    if k == "wild":
        return env
    return push(push(env, lhs[1], v[0]), lhs[2], v[1])


def prj(env, ix):
    return env[len(env) - 1 - int(ix)]


# --------------------------------------------------------------------------------------
# scalar evaluation (Interpreter.hs:898-1001)

def eval_fun(f, env, aenv):
    if isinstance(f, list) and f[0] == "lam":
        return lambda x: eval_fun(f[2], push(env, f[1], x), aenv)
    return eval_exp(f, env, aenv)


def slice_restrict(spec, slix, sh):
    """IndexSlice (Interpreter.hs:944-953); spec lists all/fixed from the innermost
    dimension outwards, mirroring SliceAll / SliceFixed nesting."""
    if not spec:
        return ()
    (slx, _i), (sl, sz) = slix, sh
    if spec[0] == "all":
        return (slice_restrict(spec[1:], slx, sl), sz)
    return slice_restrict(spec[1:], slx, sl)


def slice_extend(spec, slix, sl):
    """IndexFull (Interpreter.hs:955-965)."""
    if not spec:
        return ()
    if spec[0] == "all":
        (slx, _u), (sl1, sz) = slix, sl
        return (slice_extend(spec[1:], slx, sl1), sz)
    slx, sz = slix
    return (slice_extend(spec[1:], slx, sl), sz)


def eval_exp(e, env, aenv):
    if e == "nil":
        return ()
    k = e[0]
    ev = lambda x: eval_exp(x, env, aenv)
    if k == "var":
        return prj(env, e[1])
    if k == "let":
        return eval_exp(e[3], push(env, e[1], ev(e[2])), aenv)
    if k == "pair":
        a = ev(e[1])
        return (a, ev(e[2]))
    if k == "const":
        if vec_of(e[1]):
            return tuple(literal(vec_of(e[1])[1], t) for t in e[2])
        return literal(e[1], e[2])
    if k == "undef":
        if vec_of(e[1]):
            return tuple(literal(vec_of(e[1])[1], "0") for _ in range(vec_of(e[1])[0]))
        return literal(e[1], "0")
    if k == "vecpack":       # Interpreter.hs:942: the tuple (((), a), b) .. becomes one vector value
        parts, v = [], ev(e[3])
        while v != ():
            v, x = v
            parts.append(x)
        assert len(parts) == int(e[1])
        return tuple(parts[::-1])
    if k == "vecunpack":     # Interpreter.hs:943
        out = ()
        for x in ev(e[3]):
            out = (out, x)
        return out
    if k == "minbound":
        b = INT_BITS[e[1]]
        return -(1 << (b - 1)) if e[1][0] == "i" else 0
    if k == "maxbound":
        b = INT_BITS[e[1]]
        return (1 << (b - 1)) - 1 if e[1][0] == "i" else (1 << b) - 1
    if k == "pi":
        return fl(e[1], math.pi)
    if k == "prim":
        nty, f = PRIMS[e[1]]
        return f(*e[2:2 + nty], ev(e[2 + nty]))
    if k == "toindex":
        return to_index(ev(e[2]), ev(e[3]))
    if k == "fromindex":
        return from_index(ev(e[2]), ev(e[3]))
    if k == "indexslice":
        return slice_restrict(e[1], ev(e[2]), ev(e[3]))
    if k == "indexfull":
        return slice_extend(e[1], ev(e[2]), ev(e[3]))
    if k == "case":
        tag = ev(e[1])
        for t, rhs in e[2]:
            if int(t) == tag:
                return ev(rhs)
        if e[3] == "none":
            raise OracleError("unmatched case")
        return ev(e[3])
    if k == "cond":
        return ev(e[2]) if ev(e[1]) != 0 else ev(e[3])
    if k == "while":
        p, f, x = eval_fun(e[1], env, aenv), eval_fun(e[2], env, aenv), ev(e[3])
        while p(x) != 0:
            x = f(x)
        return x
    if k == "index":
        return prj(aenv, e[1]).index(ev(e[2]))
    if k == "linearindex":
        a = prj(aenv, e[1])
        return a.index(from_index(a.sh, ev(e[2])))
    if k == "shape":
        return prj(aenv, e[1]).sh
    if k == "shapesize":
        return size(ev(e[2]))
    if k == "foreign":
        return eval_fun(e[1], (), ())(ev(e[2]))
    if k == "coerce":
        v = ev(e[3])
        raw = np.array([v], NP[e[1]]).view(NP[e[2]])[0]
        return int(raw) if e[2] in INT_BITS else fl(e[2], raw)
    raise OracleError("unknown expression %r" % (k,))


# --------------------------------------------------------------------------------------
# array evaluation (Interpreter.hs:175-259)

def apush(aenv, lhs, v):
    return push(aenv, lhs, v)


def eval_afun(f, aenv, uses):
    if isinstance(f, list) and f[0] == "alam":
        return lambda a: eval_afun(f[2], apush(aenv, f[1], a), uses)
    return eval_acc(f, aenv, uses)


def iter_fold(n, f, c, z):
    """Shape.iter on the innermost dimension: ((z `c` f 0) `c` f 1) ..  (Shape.hs:127-132)."""
    r = z
    for i in range(n):
        r = c(r, f(i))
    return r


def iter1_fold(n, f, c):
    """Shape.iter1: f 0 `c` (f 1 `c` (.. f (n-1)))  (Shape.hs:136-142)."""
    if n == 0:
        raise OracleError("empty iteration space")
    r = f(n - 1)
    for i in range(n - 2, -1, -1):
        r = c(f(i), r)
    return r


def eval_acc(a, aenv, uses):
    if a == "anil":
        return ()
    k = a[0]
    man = lambda x: eval_acc(x, aenv, uses)
    evE = lambda x: eval_exp(x, (), aenv)
    evF = lambda x: eval_fun(x, (), aenv)
    f2 = lambda fn: (lambda x, y: fn(x)(y))

    def delayed(x):
        if isinstance(x, list) and x[0] == "delayed":
            ixf, linf = evF(x[3]), evF(x[4])
            return Delayed(x[1][2], evE(x[2]), ixf, linf)
        arr = man(x)
        return Delayed(arr.ty, arr.sh, arr.index, lambda i: arr.index(from_index(arr.sh, i)))

    if k == "avar":
        return prj(aenv, a[1])
    if k == "alet":
        return eval_acc(a[3], apush(aenv, a[1], man(a[2])), uses)
    if k == "apair":
        x = man(a[1])
        return (x, man(a[2]))
    if k == "apply":
        return eval_afun(a[1], aenv, uses)(man(a[2]))
    if k == "atrace":       # Interpreter.hs:215: evaluate the traced arrays, report, then the body
        traced = man(a[2])
        TRACE.append(("" if a[1] == "-" else bytes.fromhex(a[1]).decode(), traced))
        return man(a[3])
    if k == "aforeign":     # Interpreter.hs:217: the pure fallback in an empty environment
        return eval_afun(a[2], (), uses)(man(a[3]))
    if k == "acond":
        return man(a[2]) if evE(a[1]) != 0 else man(a[3])
    if k == "awhile":
        p, f, x = eval_afun(a[1], aenv, uses), eval_afun(a[2], aenv, uses), man(a[3])
        while p(x).read(0) != 0:
            x = f(x)
        return x
    if k == "use":
        return uses[int(a[2])]
    if k == "unit":
        v = evE(a[2])
        return from_function((), a[1], lambda ix: v)
    if k == "reshape":
        arr, sh = man(a[3]), evE(a[2])
        if size(sh) != size(arr.sh):
            raise OracleError("shape mismatch")
        return Arr(sh, arr.ty, arr.bufs)
    if k == "generate":
        return from_function(evE(a[2]), a[1][2], evF(a[3]))
    if k == "transform":
        p, f, d = evF(a[3]), evF(a[4]), delayed(a[5])
        return from_function(evE(a[2]), a[1][2], lambda ix: f(d.ixf(p(ix))))
    if k == "backpermute":
        p, d = evF(a[3]), delayed(a[4])
        return from_function(evE(a[2]), d.ty, lambda ix: d.ixf(p(ix)))
    if k == "map":
        f, d = evF(a[2]), delayed(a[3])
        return from_function(d.sh, a[1], lambda ix: f(d.ixf(ix)))
    if k == "zipwith":
        f, d1, d2 = evF(a[2]), delayed(a[3]), delayed(a[4])
        return from_function(intersect(d1.sh, d2.sh), a[1], lambda ix: f(d1.ixf(ix))(d2.ixf(ix)))
    if k == "replicate":
        arr, slix = man(a[3]), evE(a[2])
        sh = slice_extend(a[1], slix, arr.sh)
        return from_function(sh, arr.ty, lambda ix: arr.index(slice_restrict(a[1], slix, ix)))
    if k == "slice":
        arr, slix = man(a[2]), evE(a[3])
        sl = slice_restrict(a[1], slix, arr.sh)
        return from_function(sl, arr.ty, lambda ix: arr.index(_slice_full_index(a[1], slix, ix, arr.sh)))
    if k == "fold":
        f, d = f2(evF(a[1])), delayed(a[3])
        sh, n = d.sh
        if a[2] == "nothing":
            if n <= 0:
                raise OracleError("empty array")
            return from_function(sh, d.ty, lambda ix: iter1_fold(n, lambda i: d.ixf((ix, i)), f))
        z = evE(a[2][1])
        return from_function(sh, d.ty, lambda ix: iter_fold(n, lambda i: d.ixf((ix, i)), f, z))
    if k == "foldseg":
        f, d, s = f2(evF(a[2])), delayed(a[4]), delayed(a[5])
        sh, _ = d.sh
        ((), n) = s.sh
        if n <= 0:
            raise OracleError("empty segment descriptor")
        seeded = a[3] != "nothing"
        z = evE(a[3][1]) if seeded else None

        def seg_at(ix):
            sz, j = ix
            start, end = s.linf(j), s.linf(j + 1)
            if seeded:
                if end < start:
                    raise OracleError("empty segment")
                return iter_fold(end - start, lambda i: d.ixf((sz, start + i)), f, z)
            if end <= start:
                raise OracleError("empty segment")
            return iter1_fold(end - start, lambda i: d.ixf((sz, start + i)), f)
        return from_function((sh, n - 1), d.ty, seg_at)
    if k == "scan":
        return scan_op(a[1], f2(evF(a[2])), None if a[3] == "nothing" else evE(a[3][1]),
                       a[3] != "nothing", delayed(a[4]))
    if k == "scan'":
        return scan_prime_op(a[1], f2(evF(a[2])), evE(a[3]), delayed(a[4]))
    if k == "permute":
        f, dfl, p, d = f2(evF(a[1])), man(a[2]), evF(a[3]), delayed(a[4])
        out = Arr(dfl.sh, dfl.ty, [b.copy() for b in dfl.bufs])
        for src in indices(d.sh):
            tag, rest = p(src)
            if tag == 0:
                continue
            if tag != 1:
                raise OracleError("unexpected tag")
            ((), dst) = rest
            i, j = to_index(d.sh, src), to_index(out.sh, dst)
            out.write(j, f(d.linf(i), out.read(j)))
        return out
    if k == "stencil":
        f, d = evF(a[3]), delayed(a[5])
        get = bounded(a[4], d, aenv)
        return from_function(d.sh, a[2], lambda ix: f(stencil_access(a[1], get, ix)))
    if k == "stencil2":
        f, d1, d2 = evF(a[4]), delayed(a[6]), delayed(a[8])
        g1, g2 = bounded(a[5], d1, aenv), bounded(a[7], d2, aenv)
        return from_function(intersect(d1.sh, d2.sh), a[3],
                             lambda ix: f(stencil_access(a[1], g1, ix))(stencil_access(a[2], g2, ix)))
    raise OracleError("unknown array term %r" % (k,))


def _slice_full_index(spec, slix, ix, sh):
    """sliceOp's index map (Interpreter.hs:337-350): fixed dimensions take the slice
    index (bounds-checked), 'all' dimensions take the next component of ix."""
    if not spec:
        return ()
    (slx, i), (sh1, sz) = slix, sh
    if spec[0] == "all":
        ix1, j = ix
        return (_slice_full_index(spec[1:], slx, ix1, sh1), j)
    if not (0 <= i < sz):
        raise OracleError("index out of bounds")
    return (_slice_full_index(spec[1:], slx, ix, sh1), i)


def scan_op(direction, f, z, seeded, d):
    """scanlOp / scanl1Op / scanrOp / scanr1Op (Interpreter.hs:427-474, 506-552)."""
    sh, n = d.sh
    m = n + 1 if seeded else n
    out = Arr((sh, m), d.ty)
    for sz in indices(sh):
        base = to_index(sh, sz) * m
        if direction == "l":
            for i in range(m):
                if i == 0:
                    v = z if seeded else d.ixf((sz, 0))
                else:
                    v = f(out.read(base + i - 1), d.ixf((sz, i - 1 if seeded else i)))
                out.write(base + i, v)
        else:
            for i in range(m):
                if i == 0:
                    v = z if seeded else d.ixf((sz, n - 1))
                    out.write(base + m - 1, v)
                elif seeded:
                    out.write(base + n - i, f(d.ixf((sz, n - i)), out.read(base + n - i + 1)))
                else:
                    out.write(base + n - i - 1, f(d.ixf((sz, n - i - 1)), out.read(base + n - i)))
    return out


def scan_prime_op(direction, f, z, d):
    """scanl'Op / scanr'Op (Interpreter.hs:477-503, 555-582): (exclusive scan, totals)."""
    sh, n = d.sh
    out, tot = Arr((sh, n), d.ty), Arr(sh, d.ty)
    for sz in indices(sh):
        base, r = to_index(sh, sz) * n, to_index(sh, sz)
        acc = z
        for i in range(n):
            if direction == "l":
                out.write(base + i, acc)
                acc = f(acc, d.ixf((sz, i)))
            else:
                out.write(base + n - 1 - i, acc)
                acc = f(d.ixf((sz, n - 1 - i)), acc)
        tot.write(r, acc)
    return (out, tot)


def stencil_access(sr, rf, ix):
    """stencilAccess (Interpreter.hs:670-794): the outermost tuple walks the left-most
    index component; offsets run -k..+k left to right."""
    kind = sr[0]
    width = int(kind[4:]) if kind.startswith("unit") else int(kind[3:])
    k = width // 2
    if kind.startswith("unit"):
        z, i = ix
        out = ()
        for d in range(-k, k + 1):
            out = (out, rf((z, i + d)))
        return out
    dims = sh_list(ix)
    i, rest = dims[0], sh_of(dims[1:])
    out = ()
    for d, sub in zip(range(-k, k + 1), sr[1:]):
        rf2 = (lambda dd: lambda ds: rf(sh_of([i + dd] + sh_list(ds))))(d)
        out = (out, stencil_access(sub, rf2, rest))
    return out


def bounded(bnd, d, aenv):
    """bounded (Interpreter.hs:797-839)."""
    dims = sh_list(d.sh)
    kind = bnd if isinstance(bnd, str) else bnd[0]
    if kind == "constant":
        cval = eval_exp(bnd[1], (), aenv)
    if kind == "function":
        g = eval_fun(bnd[1], (), aenv)

    def get(ix):
        idx = sh_list(ix)
        if all(0 <= i < n for i, n in zip(idx, dims)):
            return d.ixf(ix)
        if kind == "function":
            return g(ix)
        if kind == "constant":
            return cval
        out = []
        for iz, sz in zip(idx, dims):
            if iz < 0:
                iz = {"clamp": 0, "mirror": -iz, "wrap": sz + iz}[kind]
            elif iz >= sz:
                iz = {"clamp": sz - 1, "mirror": sz - (iz - sz + 2), "wrap": iz - sz}[kind]
            out.append(iz)
        return d.ixf(sh_of(out))
    return get


# --------------------------------------------------------------------------------------
# entry points (Interpreter.hs:93-126)

def to_arr(a, aty):
    """numpy array(s) -> Arr.  A tuple-typed array takes a list of numpy arrays, one per
    leaf, all with the array's shape."""
    ty = aty[2]
    lv = leaves(ty)
    parts = [a] if not isinstance(a, (list, tuple)) else list(a)
    assert len(parts) == len(lv), "one buffer per scalar leaf"
    if lv:      # a vector leaf carries its components in one more, innermost numpy dimension
        dims = [int(x) for x in np.asarray(parts[0]).shape]
        shp = sh_of(dims[:-1] if vec_of(lv[0]) else dims)
    else:
        shp = sh_of(a)
    bufs = []
    for p, t in zip(parts, lv):
        v = vec_of(t)
        bufs.append(np.ascontiguousarray(p, NP[v[1]]).reshape(-1, v[0]).copy() if v
                    else np.ascontiguousarray(p, NP[t]).reshape(-1).copy())
    return Arr(shp, ty, bufs)


def from_arr(arr):
    dims = sh_list(arr.sh)
    outs = [b.reshape(dims + [vec_of(t)[0]] if vec_of(t) else dims) for b, t in zip(arr.bufs, leaves(arr.ty))]
    return outs[0] if len(outs) == 1 else outs


def _lhs_types(lhs):
    if lhs[0] == "single":
        return lhs[1]
    if lhs[0] == "wild":
        return lhs[1]
    return ("pair", _lhs_types(lhs[1]), _lhs_types(lhs[2]))


def _args_to_arrs(ty, v):
    if ty == "unit":
        return ()
    if ty[0] == "array":
        return v if isinstance(v, Arr) else to_arr(v, ty)
    return (_args_to_arrs(ty[1], v[0]), _args_to_arrs(ty[2], v[1]))


def _result_out(v):
    if isinstance(v, Arr):
        return from_arr(v)
    if v == ():
        return ()
    return (_result_out(v[0]), _result_out(v[1]))


def run_n(program_text, *args, uses=()):
    """runN: apply the program to numpy inputs, return numpy outputs (nested pairs for
    tuple results)."""
    f = parse(program_text)
    aenv = ()
    args = list(args)
    while isinstance(f, list) and f[0] == "alam":
        aenv = apush(aenv, f[1], _args_to_arrs(_lhs_types(f[1]), args.pop(0)))
        f = f[2]
    assert not args, "too many arguments"
    return _result_out(eval_acc(f, aenv, list(uses)))

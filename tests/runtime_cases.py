"""Array-level control-flow programs: alet sharing, tuples of arrays, acond, awhile, apply,
use, unit, reshape, nested manifest operands (AST.hs:235-311, Interpreter.hs:207-245)."""
from __future__ import annotations

import numpy as np

from accelerate_amd import ir as A
from accelerate_amd import programs as P

from . import progs as Q

Int = A.Int
V = lambda t: A.tarray(1, t)


def jacobi_awhile(iters):
    """awhile (\\(_, k) -> unit (k < iters)) (\\(g, k) -> (stencil g, k + 1)) (g0, unit 0), then
    the grid: the loop state is a pair (grid, Scalar Int) (Language.hs:1265-1274)."""
    ty = A.f32
    grid, cnt = A.tarray(2, ty), A.tarray(0, Int)
    state = A.tpair(A.tpair(A.unit, grid), cnt)

    def cond(st):
        (_, _g), k = st
        return A.unit_(A.u8, A.lt(Int, A.index(k, A.nil), A.constI(iters)))

    def body(st):
        (_, g), k = st
        # the applied function is built here, in the scope where it is used: its parameter's
        # de Bruijn level counts the variables bound around it
        return A.apair(A.apair(A.anil, A.apply(P.jacobi_step(), g)),
                       A.unit_(Int, A.add(Int, A.index(k, A.nil), A.constI(1))))

    def prog(g0):
        loop = A.awhile(state, cond, body, A.apair(A.apair(A.anil, g0), A.unit_(Int, A.constI(0))))
        return A.alet(state, loop, lambda st: st[0][1])

    return A.alam([grid], prog)


def runtime_cases():
    """(id, program, args, uses) with uses = [(numpy array, array type)] for (use ..) slots."""
    rng = np.random.default_rng(5)
    out = []
    add = lambda *c: out.append(c)
    x = rng.integers(-100, 100, 500).astype(np.int64)
    y = rng.integers(-100, 100, 400).astype(np.int64)

    # let-bound array used twice: sum of squares next to the plain sum, as a pair of results
    def shared(xs):
        sq = A.map_(Int, A.lam([Int], lambda v: A.mul(Int, v, v)), xs)
        return A.alet(V(Int), sq, lambda s: A.apair(
            A.fold(Q.binop(A.add, Int), A.constI(0), s),
            A.zipwith(Int, Q.binop(A.sub, Int), s, xs)))
    add("alet_shared_pair", A.alam([V(Int)], shared), [x], [])

    # acond on the host: choose a branch by comparing two extents
    def cond_prog(xs, ys):
        n, m = A.untup_shape(xs)[0], A.untup_shape(ys)[0]
        return A.acond(A.gt(Int, n, m), A.map_(Int, A.lam([Int], lambda v: A.neg(Int, v)), xs), ys)
    add("acond_true", A.alam([V(Int), V(Int)], cond_prog), [x, y], [])
    add("acond_false", A.alam([V(Int), V(Int)], cond_prog), [y, x], [])

    # a scalar the host can follow (unit of index arithmetic): returned as a result, read by a
    # kernel, fed into another such scalar, and deciding an acond
    def host_scalars(xs):
        n = A.untup_shape(xs)[0]
        S0 = A.tarray(0, Int)
        k = A.unit_(Int, A.add(Int, A.mul(Int, n, A.constI(3)), A.constI(-7)))
        return A.alet(S0, k, lambda kv: A.alet(
            S0, A.unit_(Int, A.sub(Int, A.index(kv, A.nil), A.constI(1000))), lambda k2: A.apair(
                A.apair(kv, k2),
                A.acond(A.gt(Int, A.index(k2, A.nil), A.constI(0)),
                        A.map_(Int, A.lam([Int], lambda v: A.add(Int, v, A.index(kv, A.nil))), xs),
                        A.map_(Int, A.lam([Int], lambda v: A.sub(Int, v, A.index(k2, A.nil))), xs)))))
    add("host_scalars_big", A.alam([V(Int)], host_scalars), [x], [])
    add("host_scalars_small", A.alam([V(Int)], host_scalars), [x[:20]], [])

    # acond whose predicate reads array contents (evaluated by a one-thread kernel)
    def cond_data(xs):
        first = A.index(xs, A.sh(0))
        return A.acond(A.lt(Int, first, A.constI(0)), A.scan("l", Q.binop(A.add, Int), None, xs),
                       A.scan("r", Q.binop(A.add, Int), None, xs))
    add("acond_reads_array", A.alam([V(Int)], cond_data), [x], [])

    # awhile: double every element until the total exceeds a bound
    def grow(xs):
        def cond(a):
            tot = A.fold(Q.binop(A.add, Int), A.constI(0), a)
            return A.alet(A.tarray(0, Int), tot, lambda t: A.unit_(A.u8, A.lt(Int, A.index(t, A.nil), A.constI(5000))))
        body = lambda a: A.map_(Int, A.lam([Int], lambda v: A.mul(Int, v, A.constI(2))), a)
        return A.awhile(V(Int), cond, body, xs)
    add("awhile_grow", A.alam([V(Int)], grow), [np.abs(x[:50]) + 1], [])

    # use: an embedded array (slot 0) zipped with the argument
    add("use_slot", A.alam([V(Int)], lambda xs: A.zipwith(Int, Q.binop(A.add, Int), xs, A.use(V(Int), 0))),
        [x], [(y, V(Int))])

    # reshape shares the payload; then fold the new innermost dimension
    def reshaped(xs):
        return A.fold(Q.binop(A.add, Int), A.constI(0), A.reshape(2, A.sh(25, 20), xs))
    add("reshape_then_fold", A.alam([V(Int)], reshaped), [x], [])

    # nested manifest operand: a scan consumed directly by a fold (not let-bound, Fusion.hs:552-566)
    add("fold_of_scan", A.alam([V(Int)], lambda xs: A.fold(
        Q.binop(A.max_, Int), None, A.scan("l", Q.binop(A.add, Int), None, xs))), [x], [])

    # generate whose extent depends on a scalar array (the n / shape idiom), unit + index
    def iota(n_arr):
        n = A.index(n_arr, A.nil)
        return A.generate(A.tarray(2, Int), A.sh(n, A.add(Int, n, A.constI(2))), A.lam(
            [A.tshape(2)], lambda ix: A.add(Int, A.mul(Int, A.untup(ix)[0], A.constI(100)), A.untup(ix)[1])))
    add("generate_dynamic_extent", A.alam([A.tarray(0, Int)], iota), [np.array(7, np.int64)], [])

    # atrace: the traced arrays are evaluated and reported, the result is the body's
    def traced(xs):
        return A.atrace("partial sums", A.apair(A.scan("l", Q.binop(A.add, Int), None, xs), A.unit_(Int, A.constI(7))),
                        A.map_(Int, A.lam([Int], lambda v: A.add(Int, v, A.constI(1))), xs))
    add("atrace_reports_then_continues", A.alam([V(Int)], traced), [x], [])

    # aforeign: no foreign implementation for this backend, so the pure fallback runs -- a closed
    # function applied to the evaluated argument (a fold nested under it, an outer variable unused)
    fallback = A.alam([V(Int)], lambda a: A.map_(Int, A.lam([Int], lambda v: A.mul(Int, v, A.constI(3))), a))
    add("aforeign_runs_the_fallback", A.alam([V(Int), V(Int)], lambda xs, ys: A.aforeign(
        "cublas_saxpy", fallback, A.zipwith(Int, Q.binop(A.add, Int), xs, ys))), [x, y], [])

    # permute whose defaults are a variable: the caller's array must not change
    sh1 = A.tshape(1)
    keep = A.alam([V(Int), V(Int)], lambda src, dfl: A.apair(
        A.permute(Q.binop(A.add, Int), dfl, A.lam([sh1], lambda ix: A.just(A.sh(
            A.band(Int, A.untup(ix)[0], A.constI(7))))), src), dfl))
    add("permute_copies_variable_defaults", keep, [x, np.arange(8, dtype=np.int64)], [])
    return out

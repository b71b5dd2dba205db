"""Independent pins for the oracle's array-level control flow (Interpreter.hs:207-232: Alet, Apair,
Apply, Aforeign, Acond, Awhile, Atrace, Use, Unit, Reshape).

The GPU suite compares every program of tests/runtime_cases.py with the oracle; here the oracle's
answer for each of them is checked against the same computation written directly in numpy /
Python loops -- nothing below calls into the oracle to obtain an expected value.  What each case
would catch: a do-while instead of a while (an input whose predicate is false at entry), a
fallback of Aforeign that sees the caller's environment, an Apply that binds its argument at the
wrong de Bruijn level, an Atrace that forgets to evaluate or to report, a Use that reads the wrong
slot, an Acond with its branches swapped.
"""
import numpy as np
import pytest

from accelerate_amd import ir as A
from accelerate_amd import programs as P
from oracle import interp as O

from . import progs as Q
from .cases import same
from .runtime_cases import jacobi_awhile, runtime_cases

Int = A.Int
V = lambda t: A.tarray(1, t)
CASES = {c[0]: c for c in runtime_cases()}


def _run(name):
    _, prog, args, uses = CASES[name]
    return O.run_n(prog.text(), *args, uses=[O.to_arr(u, t) for u, t in uses]), args, uses


def test_every_runtime_case_has_a_pin_here():
    pinned = {"alet_shared_pair", "acond_true", "acond_false", "host_scalars_big", "host_scalars_small",
              "acond_reads_array", "awhile_grow", "use_slot", "reshape_then_fold", "fold_of_scan",
              "generate_dynamic_extent", "atrace_reports_then_continues", "aforeign_runs_the_fallback",
              "permute_copies_variable_defaults"}
    assert set(CASES) <= pinned, sorted(set(CASES) - pinned)


def test_alet_shares_and_apair_pairs():
    got, (x,), _ = _run("alet_shared_pair")
    assert same(got, [np.array(np.sum(x * x)), x * x - x])


def test_acond_picks_by_the_predicate():
    got, (x, y), _ = _run("acond_true")      # 500 > 400: the negated first argument
    assert same(got, -x)
    got, (y2, x2), _ = _run("acond_false")   # 400 > 500 fails: the second argument as it is
    assert same(got, x2)


@pytest.mark.parametrize("name", ["host_scalars_big", "host_scalars_small"])
def test_units_of_index_arithmetic(name):
    got, (x,), _ = _run(name)
    k = 3 * len(x) - 7
    k2 = k - 1000
    third = x + k if k2 > 0 else x - k2
    assert same(got, ((np.array(k), np.array(k2)), third))


def test_acond_whose_predicate_reads_an_array():
    got, (x,), _ = _run("acond_reads_array")
    want = np.cumsum(x) if x[0] < 0 else np.cumsum(x[::-1])[::-1]
    assert same(got, want)
    # and the other branch, by flipping the first element's sign
    _, prog, _, _ = CASES["acond_reads_array"]
    z = x.copy()
    z[0] = -z[0] if z[0] != 0 else -1
    want = np.cumsum(z) if z[0] < 0 else np.cumsum(z[::-1])[::-1]
    assert same(O.run_n(prog.text(), z), want)


def _grow(a):
    n = 0
    while a.sum() < 5000:      # the test comes first: Interpreter.hs:222-229
        a = a * 2
        n += 1
    return a, n


def test_awhile_tests_before_it_steps():
    got, (x,), _ = _run("awhile_grow")
    want, steps = _grow(x.copy())
    assert steps >= 1 and same(got, want)
    # a state that fails the predicate at entry comes back untouched (a do-while would double it)
    _, prog, _, _ = CASES["awhile_grow"]
    big = np.full(50, 1000, np.int64)
    assert big.sum() >= 5000
    assert same(O.run_n(prog.text(), big), big)
    # exactly one step from just under the bound
    one = np.full(50, 99, np.int64)       # 4950 < 5000 -> 9900
    assert same(O.run_n(prog.text(), one), one * 2)


def test_awhile_over_a_pair_state_counts_its_iterations():
    # the loop state is ((grid), counter); the function applied inside is a closed Apply
    rng = np.random.default_rng(11)
    g = rng.random((6, 9)).astype(np.float32)

    def sweep(a):
        p = np.pad(a, 1, mode="edge")
        t, b, l, r = p[:-2, 1:-1], p[2:, 1:-1], p[1:-1, :-2], p[1:-1, 2:]
        return np.float32(0.25) * (((t + l) + r) + b)

    for iters in (0, 1, 5):
        want = g
        for _ in range(iters):
            want = sweep(want)
        assert same(O.run_n(jacobi_awhile(iters).text(), g), want), iters


def test_use_reads_its_slot():
    got, (x,), uses = _run("use_slot")
    y = uses[0][0]
    assert same(got, x[:len(y)] + y)      # zipWith over the intersection of the extents
    # two slots: the numbers are not interchangeable
    prog = A.alam([V(Int)], lambda xs: A.zipwith(Int, Q.binop(A.sub, Int), A.use(V(Int), 1),
                                                 A.zipwith(Int, Q.binop(A.mul, Int), xs, A.use(V(Int), 0))))
    a = np.arange(1, 9, dtype=np.int64)
    u0, u1 = a * 10, a * 1000
    got = O.run_n(prog.text(), a, uses=[O.to_arr(u0, V(Int)), O.to_arr(u1, V(Int))])
    assert same(got, u1 - a * u0)


def test_reshape_keeps_the_row_major_payload():
    got, (x,), _ = _run("reshape_then_fold")
    assert same(got, x.reshape(25, 20).sum(axis=1))


def test_a_manifest_operand_nested_in_a_consumer():
    got, (x,), _ = _run("fold_of_scan")
    assert same(got, np.array(np.cumsum(x).max()))


def test_generate_with_an_extent_from_a_scalar_array():
    got, (n,), _ = _run("generate_dynamic_extent")
    n = int(n)
    i, j = np.meshgrid(np.arange(n), np.arange(n + 2), indexing="ij")
    assert same(got, (100 * i + j).astype(np.int64))


def test_atrace_evaluates_reports_and_continues():
    del O.TRACE[:]
    got, (x,), _ = _run("atrace_reports_then_continues")
    assert same(got, x + 1)                          # the body's value
    assert len(O.TRACE) == 1
    msg, traced = O.TRACE[0]
    assert msg == "partial sums"                     # the text, decoded
    assert same(O._result_out(traced), (np.cumsum(x), np.array(7)))   # the traced arrays, evaluated
    del O.TRACE[:]


def test_aforeign_runs_a_closed_fallback():
    got, (x, y), _ = _run("aforeign_runs_the_fallback")
    assert same(got, 3 * (x[:len(y)] + y))
    # the fallback is closed (Interpreter.hs:217 evaluates it in an empty environment): one that
    # mentions a variable of the caller is an error, not a silent capture
    leaky = A.alam([V(Int), V(Int)], lambda xs, ys: A.aforeign(
        "f", A.alam([V(Int)], lambda a: A.zipwith(Int, Q.binop(A.add, Int), a, ys)), xs))
    with pytest.raises(Exception):
        O.run_n(leaky.text(), x, y)


def test_apply_binds_its_argument_innermost():
    # (\a -> zipWith (-) a ys) applied to (map (*2) xs), under two outer variables: a wrong
    # de Bruijn level would subtract the wrong array (or the argument from itself)
    x = np.arange(10, dtype=np.int64) * 7
    y = np.arange(10, dtype=np.int64) ** 2
    prog = A.alam([V(Int), V(Int)], lambda xs, ys: A.apply(
        A.alam([V(Int)], lambda a: A.zipwith(Int, Q.binop(A.sub, Int), a, ys)),
        A.map_(Int, A.lam([Int], lambda v: A.mul(Int, v, A.constI(2))), xs)))
    assert same(O.run_n(prog.text(), x, y), 2 * x - y)
    # a function of two-element scope: applied to a pair of arrays
    pair_t = A.tpair(A.tpair(A.unit, V(Int)), V(Int))
    prog2 = A.alam([V(Int), V(Int)], lambda xs, ys: A.apply(
        A.alam([pair_t], lambda st: A.zipwith(Int, Q.binop(A.sub, Int), st[0][1], st[1])),
        A.apair(A.apair(A.anil, ys), xs)))
    assert same(O.run_n(prog2.text(), x, y), y - x)


def test_permute_leaves_variable_defaults_alone():
    got, (x, d), _ = _run("permute_copies_variable_defaults")
    want = d.copy()
    np.add.at(want, np.arange(len(x)) & 7, x)
    assert same(got, [want, d])

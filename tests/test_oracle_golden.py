"""Pins the oracle (oracle/interp.py and oracle/configs.c) without a GPU:
  * against every known-answer vector the reference's doctests and regression tests hold for
    the hot path (tests/golden/vectors.json);
  * against closed forms and brute force on tiny inputs, chosen so that a dropped term, a
    wrong operand order or a transposed index fails;
  * the C loops against the Python interpreter on random inputs.
"""
import itertools

import numpy as np
import pytest

from accelerate_amd import ir as A
from accelerate_amd import programs as P
from accelerate_amd import workloads as W
from oracle import c as OC
from oracle import interp as O

from . import progs as Q
from .cases import golden_cases, same

GOLDEN = golden_cases()


@pytest.mark.parametrize("case", GOLDEN, ids=[c[0] for c in GOLDEN])
def test_interp_reproduces_reference_vectors(case):
    _, prog, args, expected = case
    assert same(O.run_n(prog.text(), *args), expected)


# ---- fold: order of operands, seed applied once and first ------------------------------------

def test_fold_is_left_fold_from_seed():
    # f acc x = 2*acc + x is not associative: only the reference's exact nesting
    # ((z `f` x0) `f` x1) .. gives this value (Shape.hs:127-132)
    f = A.lam([A.Int, A.Int], lambda a, x: A.add(A.Int, A.mul(A.Int, A.constI(2), a), x))
    prog = A.alam([A.tarray(1, A.Int)], lambda xs: A.fold(f, A.constI(1), xs))
    xs = np.array([3, 5, 7], np.int64)
    assert O.run_n(prog.text(), xs) == 2 * (2 * (2 * 1 + 3) + 5) + 7


def test_fold1_is_right_nested():
    # iter1: x0 `f` (x1 `f` x2)  (Shape.hs:136-142)
    f = A.lam([A.Int, A.Int], lambda a, x: A.sub(A.Int, a, x))
    prog = A.alam([A.tarray(1, A.Int)], lambda xs: A.fold(f, None, xs))
    assert O.run_n(prog.text(), np.array([10, 4, 1], np.int64)) == 10 - (4 - 1)


def test_fold_empty_rows_yield_seed_and_fold1_empty_is_error():
    m = np.zeros((3, 0), np.int32)
    assert same(O.run_n(P.fold_sum(A.i32, 2, 42).text(), m), np.full(3, 42, np.int32))
    with pytest.raises(O.OracleError):
        O.run_n(P.fold1_op(A.add, A.i32, 2).text(), m)


def test_int32_wraps():
    x = np.array([2**31 - 1, 1], np.int32)
    assert O.run_n(P.fold_sum(A.i32, 1, 0).text(), x) == -2**31


# ---- scans: all six against Data.List-style references on random small inputs ---------------

def _scan_ref(xs, z, direction, kind):
    f = lambda a, b: a + b
    out = []
    seq = list(xs) if direction == "l" else list(xs)[::-1]
    acc = z
    if kind == "scan1":
        for i, x in enumerate(seq):
            acc = x if i == 0 else acc + x
            out.append(acc)
        tot = None
    else:
        out.append(z)
        for x in seq:
            acc = f(acc, x)
            out.append(acc)
        tot = out[-1]
        if kind == "scan'":
            out = out[:-1]
    if direction == "r":
        out = out[::-1]
    return out, tot


@pytest.mark.parametrize("direction,kind,n", list(itertools.product("lr", ["scan", "scan1", "scan'"], [0, 1, 7])))
def test_scans_match_list_semantics(direction, kind, n):
    rng = np.random.default_rng(n)
    xs = rng.integers(-50, 50, n).astype(np.int64)
    if kind == "scan1" and n == 0:
        return
    prog = {"scan": P.scan_sum, "scan'": P.scan_prime_sum}.get(kind)
    text = (prog(direction, A.Int, 1, 5) if prog else P.scan1_sum(direction, A.Int, 1)).text()
    got = O.run_n(text, xs)
    ref, tot = _scan_ref([int(v) for v in xs], 5, direction, kind)
    if kind == "scan'":
        assert same(got, (np.array(ref, np.int64), np.array(tot, np.int64)))
    else:
        assert same(got, np.array(ref, np.int64))


def test_right_scan_puts_input_on_the_left():
    # scanr f z with f x acc = x - acc: [a - (b - (c - z)), b - (c - z), c - z, z]
    f = A.lam([A.Int, A.Int], lambda x, acc: A.sub(A.Int, x, acc))
    prog = A.alam([A.tarray(1, A.Int)], lambda xs: A.scan("r", f, A.constI(100), xs))
    a, b, c = 7, 20, 3
    assert same(O.run_n(prog.text(), np.array([a, b, c], np.int64)),
                np.array([a - (b - (c - 100)), b - (c - 100), c - 100, 100], np.int64))


def test_interval_monoid_scans():
    # non-commutative: result i = (first of element 0, second of element i)
    xs = [np.arange(5, dtype=np.int64), np.arange(5, dtype=np.int64) * 10]
    got = O.run_n(Q.interval_scan("l", "scan1").text(), xs)
    assert same(got, [np.zeros(5, np.int64), np.arange(5, dtype=np.int64) * 10])
    got = O.run_n(Q.interval_scan("r", "scan1").text(), xs)
    assert same(got, [np.arange(5, dtype=np.int64), np.full(5, 40, np.int64)])


# ---- foldSeg ---------------------------------------------------------------------------------

def test_foldseg_sum_invariant_and_empty_segments():
    rng = np.random.default_rng(5)
    lens = np.array([3, 0, 0, 5, 1, 0], np.int32)
    vals = rng.integers(-9, 9, int(lens.sum())).astype(np.int32)
    got = O.run_n(P.foldseg_sum(A.i32, A.i32, 1, 0).text(), vals, lens)
    assert got.sum() == vals.sum() and got[1] == 0 and got[2] == 0 and got[4] == vals[8]
    got7 = O.run_n(P.foldseg_sum(A.i32, A.i32, 1, 7).text(), vals, lens)
    assert same(got7, got + 7)  # the seed enters every segment exactly once, empty ones included


def test_foldseg_empty_descriptor_is_error():
    prog = A.alam([A.tarray(1, A.i32), A.tarray(1, A.i32)], lambda v, offs: A.foldseg(
        A.i32, Q.binop(A.add, A.i32), A.const(A.i32, 0), v, offs))
    with pytest.raises(O.OracleError):
        O.run_n(prog.text(), np.zeros(3, np.int32), np.zeros(0, np.int32))


# ---- permute ---------------------------------------------------------------------------------

def test_permute_new_value_is_first_argument_and_nothing_drops():
    # f new old = new - old, visited in source order (Interpreter.hs:610-619)
    f = A.lam([A.Int, A.Int], lambda new, old: A.sub(A.Int, new, old))
    sh1 = A.tshape(1)
    prog = A.alam([A.tarray(1, A.Int), A.tarray(1, A.Int)], lambda xs, dfl: A.permute(
        f, dfl, A.lam([sh1], lambda ix: A.cond(
            A.eq(A.Int, A.untup(ix)[0], A.constI(1)), A.nothing(sh1), A.just(A.sh(0)))), xs))
    got = O.run_n(prog.text(), np.array([10, 99, 3], np.int64), np.array([1, 5], np.int64))
    assert same(got, np.array([3 - (10 - 1), 5], np.int64))


def test_histogram_matches_bincount():
    keys = W.zipf_keys(5000, 64, 1)
    assert same(O.run_n(P.histogram(64).text(), keys), np.bincount(keys, minlength=64).astype(np.int32))


# ---- stencil ---------------------------------------------------------------------------------

def _bound(i, n, kind):
    if i < 0:
        return {"clamp": 0, "mirror": -i, "wrap": n + i}[kind]
    if i >= n:
        return {"clamp": n - 1, "mirror": n - (i - n + 2), "wrap": i - n}[kind]
    return i


@pytest.mark.parametrize("kind", ["clamp", "mirror", "wrap"])
def test_stencil_3x3_brute_force(kind):
    rng = np.random.default_rng(9)
    g = rng.integers(-5, 5, (4, 6)).astype(np.int64)
    got = O.run_n(Q.stencil_weighted(A.Int, [3, 3], kind).text(), g)
    ref = np.zeros_like(g)
    for y in range(4):
        for x in range(6):
            w, acc = 0, 0
            for dy in (-1, 0, 1):          # outermost tuple component walks y, top row first
                for dx in (-1, 0, 1):
                    w += 1
                    acc += w * g[_bound(y + dy, 4, kind), _bound(x + dx, 6, kind)]
            ref[y, x] = acc
    assert same(got, ref)


def test_stencil_constant_boundary_is_whole_index():
    g = np.arange(12, dtype=np.int64).reshape(3, 4)
    got = O.run_n(Q.stencil_weighted(A.Int, [3, 3], A.constant(A.Int, 1000)).text(), g)
    # corner (0,0): taps with any coordinate outside read 1000, weights 1..9 row-major
    inside = {(0, 0): 5, (0, 1): 6, (1, 0): 8, (1, 1): 9}
    exp = sum(w * g[p] for p, w in inside.items()) + 1000 * (45 - sum(inside.values()))
    assert got[0, 0] == exp


def test_jacobi_fixed_points_and_conservation():
    const = np.full((5, 7), 3.25, np.float32)
    assert same(O.run_n(P.jacobi_step().text(), const), const)          # constants are fixed points
    ramp = (np.arange(5)[:, None] * 2.0 + np.arange(7)[None, :] * 0.5).astype(np.float32)
    assert same(O.run_n(P.jacobi_step().text(), ramp)[1:-1, 1:-1], ramp[1:-1, 1:-1])  # linear: interior fixed
    assert same(OC.jacobi_f32(ramp, 1), O.run_n(P.jacobi_step().text(), ramp))


# ---- scalar primitives: Haskell semantics that differ from C ---------------------------------

def _scalar(e):
    return O.run_n(A.unit_(A.Int, e).text())


def test_div_mod_floor_quot_rem_truncate():
    c = A.constI
    assert _scalar(A.idiv(A.Int, c(-7), c(2))) == -4 and _scalar(A.mod(A.Int, c(-7), c(2))) == 1
    assert _scalar(A.quot(A.Int, c(-7), c(2))) == -3 and _scalar(A.rem(A.Int, c(-7), c(2))) == -1
    assert _scalar(A.mod(A.Int, c(7), c(-2))) == -1


def test_round_half_even_and_minmax_ord_default():
    r = lambda v: O.run_n(A.unit_(A.Int, A.round_(A.f64, A.Int, A.const(A.f64, v))).text())
    assert [r(0.5), r(1.5), r(2.5), r(-0.5), r(-1.5)] == [0, 2, 2, 0, -2]
    nan, one = A.const(A.f32, float("nan")), A.const(A.f32, 1.0)
    mx = lambda a, b: O.run_n(A.unit_(A.f32, A.max_(A.f32, a, b)).text())
    assert np.isnan(mx(nan, one)) and mx(one, nan) == 1.0   # max x y = if x <= y then y else x


def test_cond_is_lazy_in_the_untaken_branch():
    # Issue187: a branch guarding an out-of-bounds index must not be evaluated
    prog = A.alam([A.tarray(1, A.Int)], lambda xs: A.unit_(A.Int, A.cond(
        A.const(A.u8, 1), A.constI(5), A.index(xs, A.sh(99)))))
    assert O.run_n(prog.text(), np.zeros(3, np.int64)) == 5


# ---- the C loops follow the interpreter ------------------------------------------------------

def test_c_loops_match_interpreter():
    rng = np.random.default_rng(7)
    x, y = W.uniform_f32(777, 1), W.uniform_f32(777, 2)
    assert OC.dotp_f32(x, y) == O.run_n(P.dotp().text(), x, y)           # same left fold, bit-equal
    xi = W.uniform_int(500, 3)
    assert same(OC.scanl1_i64(xi), O.run_n(P.scanl1_sum(A.i64).text(), xi))
    xf = W.uniform_f32(500, 4, 0, 1)
    assert same(OC.scanl1_f32(xf), O.run_n(P.scanl1_sum(A.f32).text(), xf))
    lens = W.segment_lengths(40, 2000, 5)
    vals = W.uniform_int(2000, 6, dtype=np.int32)
    assert same(OC.foldseg_i32(vals, lens), O.run_n(P.foldseg_sum().text(), vals, lens))
    keys = W.zipf_keys(3000, 50, 8)
    assert same(OC.histogram_i32(keys, 50), O.run_n(P.histogram(50).text(), keys))
    g = W.uniform_f32(9 * 13, 9, 0, 1).reshape(9, 13)
    step = P.jacobi_step().text()
    ref = g
    for _ in range(3):
        ref = O.run_n(step, ref)
    assert same(OC.jacobi_f32(g, 3), ref)
    m = rng.integers(-1000, 1000, (4, 33)).astype(np.int32)
    assert same(OC.fold_sum_i32(m, 42), O.run_n(P.fold_sum(A.i32, 2, 42).text(), m))


def test_all_cores_loops_agree_with_the_sequential_ones():
    # the OpenMP versions only serve as a timing baseline; integer results must still be the same
    # bits, Float32 sums the same within the benchmark's tolerance
    xi = W.uniform_int(100003, 3)
    assert same(OC.omp_scanl1(xi), OC.scanl1_i64(xi))
    xf = W.uniform_f32(100003, 4, 0, 1)
    assert np.all(np.abs(OC.omp_scanl1(xf) - np.cumsum(xf.astype(np.float64))) <= 1e-4 * np.cumsum(np.abs(xf.astype(np.float64))))
    x, y = W.uniform_f32(70001, 1), W.uniform_f32(70001, 2)
    assert abs(float(OC.omp_dotp_f32(x, y)) - float(np.dot(x.astype(np.float64), y))) <= 1e-4 * float(np.sum(np.abs(x * y)))
    lens = W.segment_lengths(400, 50000, 5)
    vals = W.uniform_int(50000, 6, dtype=np.int32)
    assert same(OC.omp_foldseg_i32(vals, OC.offsets_i32(lens)), OC.foldseg_i32(vals, lens))
    keys = W.zipf_keys(200000, 1000, 8)
    assert same(OC.omp_histogram_i32(keys, 1000), OC.histogram_i32(keys, 1000))
    g = W.uniform_f32(37 * 53, 9, 0, 1).reshape(37, 53)
    assert same(OC.omp_jacobi_f32(g, 5), OC.jacobi_f32(g, 5))
    assert OC.omp_threads() >= 1


def test_workload_generators_are_seeded_and_shaped():
    lens = W.segment_lengths(1 << 12, 1 << 19, 3)
    assert lens.sum() == 1 << 19 and lens.min() >= 0 and same(lens, W.segment_lengths(1 << 12, 1 << 19, 3))
    keys = W.zipf_keys(100000, 1 << 10, 4)
    h = np.bincount(keys, minlength=1 << 10)
    assert h[0] == h.max() and 0.1 < h[0] / 100000 < 0.25   # 1/H(1024, 1.1) is about 0.17


def test_oracle_on_whole_programs_against_numpy():
    # SMVM, filter and LSD radix sort as the reference's nofib states them, against what numpy
    # gives for the same inputs: pins the oracle on compositions of scan, permute and foldSeg
    from . import progs as Q
    rng = np.random.default_rng(11)
    segd = rng.integers(0, 6, 40).astype(np.int64)
    nnz = int(segd.sum())
    inds, vals = rng.integers(0, 30, nnz).astype(np.int64), rng.integers(-9, 9, nnz).astype(np.int64)
    vec = rng.integers(-9, 9, 30).astype(np.int64)
    off = np.concatenate([[0], np.cumsum(segd)])
    ref = np.array([(vals[off[i]:off[i + 1]] * vec[inds[off[i]:off[i + 1]]]).sum() for i in range(40)])
    assert np.array_equal(O.run_n(Q.smvm(A.i64).text(), segd, inds, vals, vec), ref)
    x = rng.integers(-50, 50, 300).astype(np.int64)
    assert np.array_equal(O.run_n(Q.filter_positive().text(), x), x[x > 0])
    k = rng.integers(0, 16, 500).astype(np.int64)
    assert np.array_equal(O.run_n(Q.radix_passes(4).text(), k), np.sort(k, kind="stable"))


def test_oracle_on_segmented_scans_against_numpy():
    # scanl1Seg / scanr1Seg / scanlSeg as Prelude.hs builds them, against per-segment cumulative
    # sums: pins the oracle on scan', permute into generated defaults, and a scan over a fused zip
    from . import progs as Q
    rng = np.random.default_rng(12)
    seg = np.array([3, 0, 5, 1, 0, 0, 7, 2], np.int64)
    m = rng.integers(-9, 9, (4, 21)).astype(np.int64)     # 18 elements in segments, 3 beyond them
    off = np.concatenate([[0], np.cumsum(seg)])
    l1 = np.concatenate([np.cumsum(m[:, a:b], axis=1) for a, b in zip(off[:-1], off[1:])], axis=1)
    r1 = np.concatenate([np.cumsum(m[:, a:b][:, ::-1], axis=1)[:, ::-1] for a, b in zip(off[:-1], off[1:])], axis=1)
    assert np.array_equal(O.run_n(Q.scan1_seg("l").text(), m, seg), l1)
    assert np.array_equal(O.run_n(Q.scan1_seg("r").text(), m, seg), r1)
    z = 5
    ex = np.concatenate([np.concatenate([np.full((4, 1), z), z + np.cumsum(m[:, a:b], axis=1)], axis=1)
                         for a, b in zip(off[:-1], off[1:])], axis=1)
    got = O.run_n(Q.scanl_seg(A.i64, z).text(), m, seg)
    # the flagged scan zips with the flags of the lengthened segments: what lies beyond them is cut
    assert got.shape == (4, int(seg.sum()) + len(seg))
    assert np.array_equal(got, ex)


def test_oracle_on_issue114_and_issue409():
    # Issue114 (compared with ~= in the reference: 5e-5 absolute or 0.5 % relative for Float) and
    # Issue409, whose expected value is 1 + tanh (-1)
    import json
    import math
    import os
    from . import progs as Q
    v = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "vectors.json")))
    n, x = v["issue114"]["n"], v["issue114"]["x"]
    ef = [np.full(n, x, np.float32), np.zeros(n, np.float32)]
    close = lambda a, b: np.all((np.abs(a - b) < 5e-5) | (np.abs(a - b) <= 0.005 * np.maximum(np.abs(a), np.abs(b))))
    val, err = O.run_n(Q.issue114("fold1").text(), ef)
    assert close(val, v["issue114"]["expected_sum"][0]) and close(err, v["issue114"]["expected_sum"][1])
    vals, errs = O.run_n(Q.issue114("scanl1").text(), ef)
    assert close(vals, np.float32(x) * np.arange(1, n + 1, dtype=np.float32)) and close(errs, 0.0)
    assert O.run_n(Q.issue409(A.f64).text(), np.array(v["issue409"]["x"])) == 1 + math.tanh(-1)
    assert abs(float(O.run_n(Q.issue409(A.f32).text(), np.array(1.0, np.float32))) - (1 + math.tanh(-1))) < 1e-6


def test_oracle_on_blackscholes_against_numpy():
    # Spectral/BlackScholes.hs restated with numpy in Float64 (blackscholesRef, :96-118)
    from . import progs as Q
    rng = np.random.default_rng(13)
    p, s, y = rng.uniform(5, 30, 500), rng.uniform(1, 100, 500), rng.uniform(0.25, 10, 500)
    r, v = 0.02, 0.30

    def cnd(d):
        k = 1.0 / (1.0 + 0.2316419 * np.abs(d))
        poly = k * (0.31938153 + k * (-0.356563782 + k * (1.781477937 + k * (-1.821255978 + k * 1.330274429))))
        c = 0.39894228040143267793994605993438 * np.exp(-0.5 * d * d) * poly
        return np.where(d > 0, 1.0 - c, c)
    vs = v * np.sqrt(y)
    d1 = (np.log(p / s) + (r + 0.5 * v * v) * y) / vs
    d2 = d1 - vs
    xe = s * np.exp(-r * y)
    call, put = O.run_n(Q.blackscholes(A.f64).text(), [p, s, y])
    assert np.allclose(call, p * cnd(d1) - xe * cnd(d2), rtol=1e-12, atol=1e-12)
    assert np.allclose(put, xe * (1.0 - cnd(d2)) - p * (1.0 - cnd(d1)), rtol=1e-12, atol=1e-12)


def test_long_array_programs_at_a_small_size():
    # the programs of the GPU test over more than 2^32 elements, at a size the oracle walks:
    # their closed-form expectations are checked here
    big, n = 1000 + 5, 50
    fold, far_end, scan_end = Q.long_array_programs(big, n)
    assert int(O.run_n(fold.text())) == Q.long_fold_expected(big) == 7 + sum(i & 255 for i in range(big))
    assert same(O.run_n(far_end.text()), ((np.arange(big - 8, big) & 255) + 1).astype(np.uint8))
    assert same(O.run_n(scan_end.text()), np.arange(n - 5, n + 1).astype(np.int32))

"""Test cases shared by the CPU suite (oracle vs. the reference's known answers) and the GPU
suite (HIP backend vs. oracle and known answers)."""
from __future__ import annotations

import json
import os

import numpy as np

from accelerate_amd import ir as A
from accelerate_amd import programs as P

from . import progs as Q

HERE = os.path.dirname(os.path.abspath(__file__))
VEC = json.load(open(os.path.join(HERE, "golden", "vectors.json")))
I64 = np.int64


def _nest(parts):
    """Value (((), p0), p1) .. of the given components, outermost first."""
    v = A.nil
    for p in parts:
        v = A.pair(v, p)
    return v


def golden_cases():
    """(id, program, args, expected): expected is what the reference's own doctests /
    regression tests state (tests/golden/vectors.json)."""
    v = VEC
    out = []
    add = lambda *c: out.append(c)
    add("fold_sum_seed42", P.fold_sum(A.Int, 2, 42), [np.array(v["fold_sum_seed42"]["mat"], I64)],
        np.array(v["fold_sum_seed42"]["expected"], I64))
    add("mss", Q.mss(), [np.array(v["mss"]["vec"], I64)], np.array(v["mss"]["expected"], I64))
    add("scanl_vec", P.scan_sum("l", A.Int, 1, v["scanl_vec"]["seed"]), [np.array(v["scanl_vec"]["vec"], I64)],
        np.array(v["scanl_vec"]["expected"], I64))
    add("scanl_mat", P.scan_sum("l", A.Int, 2, 0), [np.array(v["scanl_mat"]["mat"], I64)],
        np.array(v["scanl_mat"]["expected"], I64))
    add("scanl_prime_vec", P.scan_prime_sum("l", A.Int, 1, 0), [np.array(v["scanl_prime_vec"]["vec"], I64)],
        (np.array(v["scanl_prime_vec"]["expected"], I64), np.array(v["scanl_prime_vec"]["expected_sum"], I64)))
    add("scanl_prime_mat", P.scan_prime_sum("l", A.Int, 2, 0), [np.array(v["scanl_prime_mat"]["mat"], I64)],
        (np.array(v["scanl_prime_mat"]["expected"], I64), np.array(v["scanl_prime_mat"]["expected_sum"], I64)))
    add("scanl1_mat", P.scanl1_sum(A.Int, 2), [np.array(v["scanl1_mat"]["mat"], I64)],
        np.array(v["scanl1_mat"]["expected"], I64))
    r, c = v["misc_scanl1"]["rows"], v["misc_scanl1"]["cols"]
    arr = np.arange(1, r * c + 1, dtype=I64).reshape(r, c)
    intsum = lambda n, m: m * (m + 1) // 2 - (n - 1) * n // 2
    ref = np.array([[intsum(1 + i * c, 1 + i * c + j) for j in range(c)] for i in range(r)], I64)
    add("misc_scanl1", P.scanl1_sum(A.Int, 2), [arr], ref)
    add("foldseg_doctest", P.foldseg_sum(A.Int, A.Int, 2, 0),
        [np.array(v["foldseg_doctest"]["mat"], I64), np.array(v["foldseg_doctest"]["seg"], I64)],
        np.array(v["foldseg_doctest"]["expected"], I64))
    add("histogram_doctest", P.histogram(v["histogram_doctest"]["bins"], A.Int, A.Int),
        [np.array(v["histogram_doctest"]["keys"], I64)], np.array(v["histogram_doctest"]["expected"], I64))
    add("identity_permute", Q.identity_permute(), [np.array(v["identity_permute"]["n"], I64)],
        np.array(v["identity_permute"]["expected"], I64))
    add("transpose_backpermute", Q.transpose(), [np.array(v["transpose_backpermute"]["mat"], I64)],
        np.array(v["transpose_backpermute"]["expected"], I64))
    for name, prog in (("scanlseg_doctest", Q.scanl_seg()), ("scanl1seg_doctest", Q.scan1_seg("l")),
                       ("scanr1seg_doctest", Q.scan1_seg("r"))):
        add(name, prog, [np.array(v[name]["mat"], I64), np.array(v[name]["seg"], I64)], np.array(v[name]["expected"], I64))
    # regression tests of the reference with literal answers (Test/NoFib/Issues)
    add("issue93", Q.issue93(), [np.array(v["issue93"]["mat"], I64)], np.array(v["issue93"]["expected"], I64))
    add("issue102", Q.issue102(), [], np.array(v["issue102"]["expected"], I64))
    for n in "ABCD":
        e = v["issue119_" + n]
        dt = np.int32 if e["type"] == "i32" else I64
        add("issue119_" + n, Q.issue119_foldall(e["type"]), [np.array(e["xs"], dt).reshape(e["shape"])],
            np.array(e["expected"][0], dt))
    e = v["issue119_E"]
    add("issue119_E", Q.fold_op(A.add, A.i32, 2, 0), [np.array(e["xs"], np.int32).reshape(e["shape"])],
        np.array(e["expected"], np.int32))
    for n, prog in (("F", Q.scan1_seg("l", A.i64, 1, A.i32)), ("G", Q.scan1_seg("r", A.i64, 1, A.i32)),
                    ("H", Q.scanl_seg(A.i64, 0, 1, A.i32)), ("I", Q.scanr_seg(A.i64, 0, 1, A.i32))):
        e = v["issue119_" + n]
        add("issue119_" + n, prog, [np.array(e["xs"], I64), np.array(e["seg"], np.int32)], np.array(e["expected"], I64))
    for n, d in (("J", "l"), ("K", "r")):
        e = v["issue119_" + n]
        add("issue119_" + n, Q.scan_prime_seg(d, A.i64, 0, 1, A.i32), [np.array(e["xs"], I64), np.array(e["seg"], np.int32)],
            (np.array(e["expected"], I64), np.array(e["expected_sums"], I64)))
    for name, d in (("scanlprimeseg_doctest", "l"), ("scanrprimeseg_doctest", "r")):
        e = v[name]
        add(name, Q.scan_prime_seg(d), [np.array(e["mat"], I64), np.array(e["seg"], I64)],
            (np.array(e["expected"], I64), np.array(e["expected_sums"], I64)))
    # doctests of Prelude.hs beyond the skeletons' own
    e = v["scanrseg_doctest"]
    add("scanrseg_doctest", Q.scanr_seg(A.Int, 0, 2), [np.array(e["mat"], I64), np.array(e["seg"], I64)], np.array(e["expected"], I64))
    e = v["foldall_doctest"]
    add("foldall_vec_doctest", Q.fold_all(A.f32, 1, e["seed"]), [np.array(e["vec"], np.float32)], np.array(e["expected_vec"], np.float32))
    add("foldall_mat_doctest", Q.fold_all(A.f32, 2, 0), [np.array(e["mat"], np.float32)], np.array(e["expected_mat"], np.float32))
    e = v["all_any_doctest"]
    add("fold_all_even_doctest", Q.all_any("all"), [np.array(e["mat"], I64)], np.array(e["all"], np.uint8))
    add("fold_any_even_doctest", Q.all_any("any"), [np.array(e["mat"], I64)], np.array(e["any"], np.uint8))
    e = v["reductions_doctest"]
    add("fold_sum_doctest", Q.fold_op(A.add, A.Int, 2, 0), [np.array(e["mat2x5"], I64)], np.array(e["sum"], I64))
    add("fold_product_doctest", Q.fold_op(A.mul, A.Int, 2, 1), [np.array(e["mat2x5"], I64)], np.array(e["product"], I64))
    add("fold1_minimum_doctest", Q.fold_op(A.min_, A.Int, 2), [np.array(e["mat3x4"], I64)], np.array(e["minimum"], I64))
    add("fold1_maximum_doctest", Q.fold_op(A.max_, A.Int, 2), [np.array(e["mat3x4"], I64)], np.array(e["maximum"], I64))
    e = v["prepostscanl_doctest"]
    add("scan_prescanl_doctest", Q.prescanl_sum(), [np.array(e["vec"], I64)], np.array(e["prescanl"], I64))
    add("scan_postscanl_doctest", Q.postscanl_sum(e["postscanl_seed"]), [np.array(e["vec"], I64)], np.array(e["postscanl"], I64))
    e = v["filter_doctest"]
    add("filter_even_doctest", Q.filter_even(), [np.array(e["vec"], I64)], (np.array(e["expected"], I64), np.array(e["count"], I64)))
    e = v["gather_scatter_doctest"]
    g = e["gather"]
    add("gather_doctest", Q.gather(A.Int), [np.array(g["from"], I64), np.array(g["input"], I64)], np.array(g["expected"], I64))
    g = e["gatherIf"]
    add("gatherif_doctest", Q.gather_if(), [np.array(g["from"], I64), np.array(g["mask"], I64), np.array(g["defaults"], np.float32),
                                            np.array(g["input"], np.float32)], np.array(g["expected"], np.float32))
    g = e["scatter"]
    add("scatter_doctest", Q.scatter(A.Int), [np.array(g["to"], I64), np.zeros(g["size"], I64), np.array(g["input"], I64)],
        np.array(g["expected"], I64))
    g = e["scatterIf"]
    add("scatterif_doctest", Q.scatter_if(), [np.array(g["to"], I64), np.array(g["mask"], I64), np.zeros(g["size"], I64),
                                              np.array(g["input"], I64)], np.array(g["expected"], I64))
    e = v["reindex_doctest"]
    mat, box = np.array(e["mat"], I64), np.arange(30, dtype=I64).reshape(e["box_shape"])
    last = lambda d: A.sub(A.Int, d, A.constI(1))
    add("reverseon_1_doctest", Q.reindex(2, lambda d: d(), lambda ix, d: [ix[0], A.sub(A.Int, last(d()[1]), ix[1])]),
        [mat], np.array(e["reverseOn_1"], I64))
    add("reverseon_2_doctest", Q.reindex(2, lambda d: d(), lambda ix, d: [A.sub(A.Int, last(d()[0]), ix[0]), ix[1]]),
        [mat], np.array(e["reverseOn_2"], I64))
    add("transposeon_1_2_box_doctest", Q.reindex(3, lambda d: [d()[0], d()[2], d()[1]], lambda ix, d: [ix[0], ix[2], ix[1]]),
        [box], np.array(e["transposeOn_1_2_box"], I64).reshape(2, 5, 3))
    add("transposeon_2_3_box_doctest", Q.reindex(3, lambda d: [d()[1], d()[0], d()[2]], lambda ix, d: [ix[1], ix[0], ix[2]]),
        [box], np.array(e["transposeOn_2_3_box"], I64).reshape(3, 2, 5))
    add("transposeon_1_3_box_doctest", Q.reindex(3, lambda d: [d()[2], d()[1], d()[0]], lambda ix, d: [ix[2], ix[1], ix[0]]),
        [box], np.array(e["transposeOn_1_3_box"], I64).reshape(5, 3, 2))
    add("take_5_doctest", Q.reindex(2, lambda d: [d()[0], A.min_(A.Int, A.constI(5), d()[1])], lambda ix, d: ix),
        [mat], np.array(e["take_5"], I64))
    add("drop_7_doctest", Q.reindex(2, lambda d: [d()[0], A.sub(A.Int, d()[1], A.min_(A.Int, A.constI(7), d()[1]))],
                                    lambda ix, d: [ix[0], A.add(A.Int, ix[1], A.min_(A.Int, A.constI(7), d()[1]))]),
        [mat], np.array(e["drop_7"], I64))
    add("init_doctest", Q.reindex(2, lambda d: [d()[0], last(d()[1])], lambda ix, d: ix), [mat], np.array(e["init"], I64))
    add("tail_doctest", Q.reindex(2, lambda d: [d()[0], last(d()[1])], lambda ix, d: [ix[0], A.add(A.Int, ix[1], A.constI(1))]),
        [mat], np.array(e["tail"], I64))
    e = v["concat_doctest"]
    add("append_doctest", Q.concat_on(1), [np.array(e["m1"], I64), np.array(e["m2_10x3"], I64)], np.array(e["append"], I64))
    add("concaton_1_doctest", Q.concat_on(1), [np.array(e["m1"], I64), np.array(e["m2_10x5"], I64)], np.array(e["concatOn_1"], I64))
    add("concaton_2_doctest", Q.concat_on(2), [np.array(e["m1"], I64), np.array(e["m2_10x5"], I64)], np.array(e["concatOn_2"], I64))
    e = v["replicate_slice_doctest"]
    vec, mat, cube = np.array(e["vec"], I64), np.array(e["mat"], I64), np.arange(60, dtype=I64).reshape(e["cube_shape"])
    fx, un = (lambda n: A.constI(n)), A.nil
    sl = lambda *parts: (lambda: _nest(parts))      # slice index, outermost component first
    add("replicate_4_all_doctest", Q.replicate_(("all", "fixed"), sl(fx(4), un), 1, 2), [vec], np.array(e["replicate_4_All"], I64))
    add("replicate_all_4_doctest", Q.replicate_(("fixed", "all"), sl(un, fx(4)), 1, 2), [vec], np.array(e["replicate_All_4"], I64))
    add("replicate_2_all_3_doctest", Q.replicate_(("fixed", "all", "fixed"), sl(fx(2), un, fx(3)), 1, 3), [vec],
        np.array(e["replicate_2_All_3"], I64))
    add("slice_2_all_doctest", Q.slice_of(("all", "fixed"), sl(fx(2), un), 2, 1), [mat], np.array(e["slice_2_All"], I64))
    add("slice_4_2_doctest", Q.slice_of(("fixed", "fixed"), sl(fx(4), fx(2)), 2, 0), [mat], np.array(e["slice_4_2"], I64))
    add("slice_sl0_vec_doctest", Q.slice_of(("fixed",), sl(fx(4)), 1, 0), [vec], np.array(e["sl0_vec_4"], I64))
    add("slice_sl0_mat_doctest", Q.slice_of(("fixed", "all"), sl(un, fx(4)), 2, 1), [mat], np.array(e["sl0_mat_4"], I64))
    add("slice_sl1_mat_doctest", Q.slice_of(("all", "fixed"), sl(fx(4), un), 2, 1), [mat], np.array(e["sl1_mat_4"], I64))
    add("slice_sl1_cube_doctest", Q.slice_of(("all", "fixed", "all"), sl(un, fx(2), un), 3, 2), [cube], np.array(e["sl1_cube_2"], I64))
    e = v["map_zipwith_doctest"]
    add("map_plus1_doctest", A.alam([A.tarray(1, A.Int)], lambda xs: A.map_(A.Int, A.lam([A.Int], lambda x: A.add(A.Int, x, A.constI(1))), xs)),
        [np.array(e["xs"], I64)], np.array(e["map_plus1"], I64))
    add("zipwith_plus_doctest", A.alam([A.tarray(2, A.Int)] * 2, lambda a, b: A.zipwith(A.Int, Q.binop(A.add, A.Int), a, b)),
        [np.array(e["m3x5"], I64), np.array(e["m5x10"], I64)], np.array(e["zipwith_plus"], I64))
    e = v["producers_doctest"]
    xs5 = np.array(e["indexed_vec"], np.float32)
    add("indexed_vec_doctest", Q.indexed(1), [xs5], [np.arange(5, dtype=I64), xs5])
    m34 = np.arange(12, dtype=np.float32).reshape(e["indexed_mat_shape"])
    add("indexed_mat_doctest", Q.indexed(2), [m34], [np.repeat(np.arange(3, dtype=I64), 4).reshape(3, 4),
                                                     np.tile(np.arange(4, dtype=I64), 3).reshape(3, 4), m34])
    add("enumfromn_doctest", Q.enum_from_step_n(2, (5, 10), A.Int, 0, 1), [], np.array(e["enumFromN_5x10"], I64))
    add("enumfromstepn_doctest", Q.enum_from_step_n(2, (5, 10), A.f32, 0.0, 0.5), [], np.array(e["enumFromStepN_5x10"], np.float32))
    odd = lambda x: A.neq(A.Int, A.rem(A.Int, x, A.constI(2)), A.constI(0))
    add("filter_odd_mat_doctest", Q.filter_rows(odd), [np.array(e["filter_odd_mat"], I64)],
        (np.array(e["filter_odd"], I64), np.array(e["filter_odd_counts"], I64)))
    e = v["misc_cache"]
    for which in ("generate", "backpermute"):
        add("misc_cache_" + which, Q.misc_cache(which), [np.array(e["a"], np.float32), np.array(e["b"], np.float32)],
            np.array(e[which], np.float32))
    add("issue123", Q.issue123(v["issue123"]["n"]), [], np.array(v["issue123"]["expected"], I64))
    add("issue184_A", Q.issue184a(v["issue184_A"]["n"]), [np.array(v["issue184_A"]["v"], I64)],
        np.array(v["issue184_A"]["expected"], I64))
    add("issue287_A", Q.issue287a(), [[np.zeros(v["issue287_A"]["n"], I64)] * 6],
        [np.array(c, I64) for c in zip(*v["issue287_A"]["expected"])])
    pairs = [np.arange(1, v["issue288"]["n"] + 1, dtype=I64)] * 2
    add("issue288", Q.issue288(), [pairs], pairs)
    for n in v["issue364"]["sizes"]:
        add("issue364_%d" % n, Q.issue364(), [[np.arange(n, dtype=I64)] * 2],
            [np.concatenate([[-1], np.zeros(n, I64)]), np.concatenate([[-1], np.arange(n, dtype=I64)])])
    for ty, dt in ((A.f32, np.float32), (A.f64, np.float64)):
        xs = np.array([float(t) for t in v["issue407"]["xs"]], dt)
        add("issue407_isnan_" + ty, Q.issue407("isnan", ty), [xs], np.array(v["issue407"]["isnan"], np.uint8))
        add("issue407_isinf_" + ty, Q.issue407("isinf", ty), [xs], np.array(v["issue407"]["isinf"], np.uint8))
    e = v["issue436_A"]
    add("issue436_A", Q.filter_take(e["take"]), [np.array(e["xs"], np.uint8)],
        (np.array(e["expected"], np.uint8), np.array(e["count"], I64)))
    add("issue439", Q.issue439(), [], np.array(v["issue439"]["expected"], np.float32))
    F32 = np.float32
    for which in "ABC":
        add("issue168_" + which, Q.issue168(which), [], [np.array([x], F32) for x in v["issue168"][which]])
    rng = np.random.default_rng(264)
    for ty, dt in ((A.i8, np.int8), (A.i16, np.int16), (A.i32, np.int32), (A.i64, np.int64), (A.u8, np.uint8),
                   (A.u16, np.uint16), (A.u32, np.uint32), (A.u64, np.uint64)):
        info = np.iinfo(dt)
        xs = np.concatenate([np.array([info.min, info.max, 0], dt), rng.integers(info.min, info.max, 61, dtype=dt, endpoint=True)])
        add("issue264_negneg_" + ty, Q.issue264_neg(ty), [xs], xs)
    for ty, dt in ((A.f32, np.float32), (A.f64, np.float64)):
        xs = np.concatenate([[0.0, -0.0, np.inf, -np.inf], rng.standard_normal(60)]).astype(dt)
        add("issue264_negneg_" + ty, Q.issue264_neg(ty), [xs], xs)
    table = {"not.not": lambda u: u, "not(&&)": lambda u, w: 1 - (u & w), "not(||)": lambda u, w: 1 - (u | w),
             "not(not(&&))": lambda u, w: u & w, "not(not(||))": lambda u, w: u | w}
    assert set(table) == set(v["issue264"]["bool"])
    for which, f in table.items():
        for bits in ((0,), (1,)) if which == "not.not" else ((0, 0), (0, 1), (1, 0), (1, 1)):
            add("issue264_%s_%s" % (which, "".join(map(str, bits))), Q.issue264_bool(which),
                [np.array(b, np.uint8) for b in bits], np.array(f(*bits), np.uint8))
    t = v["issue286"]
    add("issue286", Q.issue286(), [np.full(t["shape"], t["fill"], np.uint8)], np.array(t["expected"], F32))
    for shp in v["issue427"]["shapes"]:
        cells = (np.random.default_rng(427).random(shp) < 0.4).astype(np.uint8)
        add("issue427_%dx%d" % tuple(shp), Q.indices_of_truth(), [cells], [c.astype(I64) for c in np.nonzero(cells)])
    t = v["issue517"]
    add("issue517", Q.issue517(), [], [np.array(x, dt) for tag, val in zip(t["tags"], t["values"])
                                        for x, dt in ((tag, np.uint8), (0.0 if val is None else val, F32))])
    n = v["issue551"]["n"]
    add("issue551_eq", Q.issue551("eq"), [], np.eye(n, dtype=np.uint8))
    add("issue551_digits", Q.issue551("digits"), [], np.arange(n, dtype=np.uint16))
    t = v["issue228"]
    pair_in = [np.array(t["fst"], I64), np.array(t["snd"], I64)]
    pair_out = [np.array(t["expected"][0], I64), np.array(t["expected"][1], I64)]
    add("issue228_fold", Q.issue228(True), [pair_in], pair_out)
    add("issue228_fold1", Q.issue228(False), [pair_in], pair_out)
    for k in (4, 5):
        add("issue362_%dtuple" % k, Q.tuple_scanl1(k), [[np.array(v["issue362"]["vec"], I64)] * k],
            [np.array(v["issue362"]["expected"], I64)] * k)
    for name in ("issue185_A", "issue185_B"):
        t = v[name]
        add(name, Q.scatter(), [np.array(t["to"], I64), np.array(t["over"], I64), np.array(t["xs"], I64)],
            np.array(t["expected"], I64))
    t = v["issue185_E"]
    add("issue185_E", Q.gather(), [np.array(t["from"], I64), np.array(t["xs"], I64)], np.array(t["expected"], I64))
    t = v["issue137"]
    a = np.arange(1, t["size"] + 1, dtype=I64)
    exp = np.array(t["expected"], I64)
    add("issue137", Q.issue137(), [8 - (a % 17), a // 8], [exp[:, 0].copy(), exp[:, 1].copy()])
    return out


def same(a, b, exact=True, rtol=0.0, atol=0.0):
    """Structural comparison of results: nested pairs of arrays / lists of leaf arrays."""
    if isinstance(a, (tuple, list)):
        return isinstance(b, (tuple, list)) and len(a) == len(b) and all(
            same(x, y, exact, rtol, atol) for x, y in zip(a, b))
    a, b = np.asarray(a), np.asarray(b)
    if a.shape != b.shape:
        return False
    if exact:
        return bool(np.array_equal(a, b, equal_nan=True)) if a.dtype.kind == "f" else bool(np.array_equal(a, b))
    return bool(np.allclose(a, b, rtol=rtol, atol=atol, equal_nan=True))


# ------------------------------------------------------------------------------------------
# random cases shaped like the reference's property tests (Test/NoFib/Prelude/*.hs): small
# extents, every rank, empty dimensions, neutral and non-neutral seeds, non-commutative
# operators, all boundary kinds.  (id, program, args, tolerance): tolerance None = bit-exact.

NPT = {"i8": np.int8, "i16": np.int16, "i32": np.int32, "i64": np.int64, "u8": np.uint8, "u16": np.uint16,
       "u32": np.uint32, "u64": np.uint64, "f16": np.float16, "f32": np.float32, "f64": np.float64}


def _rand(rng, ty, shape, lo=-1000, hi=1000):
    if ty in A.FLOATING:
        return rng.uniform(-4, 4, shape).astype(NPT[ty])
    if ty[0] == "u":
        lo = 0
    info = np.iinfo(NPT[ty])
    return rng.integers(max(lo, info.min), min(hi, info.max), shape, endpoint=True).astype(NPT[ty])


SHAPES = {1: [(0,), (1,), (63,), (300,), (5000,)],
          2: [(3, 0), (0, 4), (5, 10), (17, 129), (2, 4100), (900, 7), (150, 33), (3000, 1)],
          3: [(2, 3, 0), (3, 4, 50), (2, 2, 700), (30, 20, 3)]}


def parity_cases():
    rng = np.random.default_rng(2024)
    out = []
    add = lambda *c: out.append(c)
    # ---- fold (Prelude/Fold.hs:42-121)
    for rank, shapes in SHAPES.items():
        for shp in shapes:
            for ty in (A.i32, A.i64):
                x = _rand(rng, ty, shp)
                add("fold_sum_%s_%s" % (ty, shp), P.fold_sum(ty, rank, 0), [x], None)
                add("fold_sum_seed_%s_%s" % (ty, shp), P.fold_sum(ty, rank, 42), [x], None)
                if shp[-1] > 0:
                    add("fold1_min_%s_%s" % (ty, shp), P.fold1_op(A.min_, ty, rank), [x], None)
                    add("fold1_max_%s_%s" % (ty, shp), P.fold1_op(A.max_, ty, rank), [x], None)
            if shp[-1] > 0:
                add("fold_mss_%s" % (shp,), Q.mss(A.Int, rank), [_rand(rng, A.i64, shp, -100, 100)], None)
            xf = _rand(rng, A.f32, shp)
            add("fold_sum_f32_%s" % (shp,), P.fold_sum(A.f32, rank, 0), [xf], 1e-4 * 4 * max(1, shp[-1]))
    # ---- scans (Prelude/Scan.hs:47-469)
    for rank, shapes in SHAPES.items():
        for shp in shapes:
            x = _rand(rng, A.i64, shp)
            pr = [_rand(rng, A.i64, shp), _rand(rng, A.i64, shp)]
            for d in "lr":
                add("scan_%s_seed_%s" % (d, shp), P.scan_sum(d, A.i64, rank, 7), [x], None)
                add("scan'_%s_%s" % (d, shp), P.scan_prime_sum(d, A.i64, rank, 0), [x], None)
                add("scan_interval_%s_%s" % (d, shp), Q.interval_scan(d, "scan", A.Int, rank), [pr], None)
                add("scan'_interval_%s_%s" % (d, shp), Q.interval_scan(d, "scan'", A.Int, rank), [pr], None)
                if shp[-1] > 0:
                    add("scan1_%s_%s" % (d, shp), P.scan1_sum(d, A.i64, rank), [x], None)
                    add("scan1_interval_%s_%s" % (d, shp), Q.interval_scan(d, "scan1", A.Int, rank), [pr], None)
        xf = _rand(rng, A.f32, shapes[-1]) + np.float32(4)
        add("scanl1_f32_%s" % (shapes[-1],), P.scanl1_sum(A.f32, rank), [xf], 1e-4 * 8 * shapes[-1][-1])
    # ---- foldSeg (Prelude/Fold.hs:102-121): both descriptor types, empty segments, outer rows
    for ity in (A.i32, A.i64):
        for shp, nseg in [((0,), 3), ((200,), 1), ((5000,), 64), ((3, 700), 9), ((2, 5, 300), 4), ((9000,), 2500)]:
            n = shp[-1]
            cuts = np.sort(rng.integers(0, n + 1, nseg - 1)) if nseg > 1 else np.array([], np.int64)
            lens = np.diff(np.concatenate([[0], cuts, [n]])).astype(NPT[ity])
            if nseg > 2:
                lens[-1] = max(0, int(lens[-1]) - 3)     # leave a few trailing elements in no segment
            v = _rand(rng, A.i32, shp)
            add("foldseg_%s_%s_%d" % (ity, shp, nseg), P.foldseg_sum(A.i32, ity, len(shp), 5), [v, lens], None)
    # ---- fold1Seg (Prelude/Fold.hs:102-121): DIM1-3, a sum and the non-commutative interval monoid,
    #      both descriptor types; no empty segment (that is an error, tested apart)
    for ity in (A.i32, A.i64):
        for shp, nseg in [((200,), 1), ((5000,), 64), ((3, 700), 9), ((2, 5, 300), 4), ((9000,), 2500), ((40000,), 3)]:
            n = shp[-1]
            cuts = np.sort(rng.choice(np.arange(1, n), nseg - 1, replace=False)) if nseg > 1 else np.array([], np.int64)
            lens = np.diff(np.concatenate([[0], cuts, [n]])).astype(NPT[ity])
            if nseg > 2 and lens[-1] > 3:
                lens[-1] -= 3                             # leave a few trailing elements in no segment
            add("fold1seg_sum_%s_%s_%d" % (ity, shp, nseg), Q.fold1seg_sum(A.i64, len(shp), ity),
                [_rand(rng, A.i64, shp), lens], None)
            add("fold1seg_interval_%s_%s_%d" % (ity, shp, nseg), Q.fold1seg_interval(len(shp), A.Int, ity),
                [[_rand(rng, A.i64, shp), _rand(rng, A.i64, shp)], lens], None)
    # ---- permute (Prelude/Permute.hs:46-146): (+) with collisions and drops, every rank pair
    for sr, dr in [(1, 1), (2, 1), (1, 2), (3, 2), (2, 3)]:
        sshape = {1: (400,), 2: (13, 31), 3: (4, 5, 21)}[sr]
        dshape = {1: (37,), 2: (5, 7), 3: (2, 3, 4)}[dr]
        nd = int(np.prod(dshape))
        to = rng.integers(-nd // 4, nd, int(np.prod(sshape))).astype(np.int64)  # negatives are dropped
        for ty in (A.i32, A.i64, A.f32):
            xs = _rand(rng, ty, sshape, -20, 20)
            if ty == A.f32:
                xs = np.round(xs * 4) / 4     # sums of quarters are exact in any order
            add("permute_add_%s_%d_%d" % (ty, sr, dr), Q.accumulate(ty, sr, dr), [xs, to, _rand(rng, ty, dshape, -5, 5)
                if ty != A.f32 else np.zeros(dshape, np.float32)], None)
    # ---- permute with a component-wise combination over pairs (one atomic per component)
    to = rng.integers(0, 29, 3000).astype(np.int64)
    quarters = lambda n: (np.round(rng.uniform(-20, 20, n) * 4) / 4).astype(np.float32)
    add("permute_pairs_f32_add_add", Q.accumulate_pairs(), [[quarters(3000), quarters(3000)], to,
                                                            [np.zeros(29, np.float32), quarters(29)]], None)
    add("permute_pairs_i64_add_i32_max", Q.accumulate_pairs(A.i64, A.i32, A.max_),
        [[_rand(rng, A.i64, (3000,)), _rand(rng, A.i32, (3000,))], to, [_rand(rng, A.i64, (29,)), _rand(rng, A.i32, (29,))]], None)
    add("permute_pairs_u32_add_u64_bxor", Q.accumulate_pairs(A.u32, A.u64, A.bxor),
        [[_rand(rng, A.u32, (3000,)), _rand(rng, A.u64, (3000,))], to, [_rand(rng, A.u32, (29,)), _rand(rng, A.u64, (29,))]], None)
    # ---- backpermute (Prelude/Backpermute.hs)
    add("transpose_33x17", Q.transpose(A.i32), [_rand(rng, A.i32, (33, 17))], None)
    add("gather", Q.gather(A.f32), [rng.integers(0, 100, 257).astype(np.int64), _rand(rng, A.f32, (100,))], None)
    # ---- stencil (Prelude/Stencil.hs:48-290): 1D/2D/3D, widths 3..9, all five boundary kinds
    for widths, shp in [([3], (1,)), ([3], (50,)), ([5], (64,)), ([7], (9,)), ([9], (300,)), ([3, 3], (1, 1)),
                        ([3, 3], (17, 40)), ([5, 5], (9, 11)), ([3, 5], (30, 70)), ([7, 7], (8, 8)),
                        ([3, 3, 3], (5, 6, 7)), ([3, 3, 3], (2, 1, 9))]:
        for bname in ("clamp", "mirror", "wrap", "constant", "function"):
            if bname == "mirror" and any(s < (w // 2) + 1 for w, s in zip(widths, shp)):
                continue    # mirror needs extent > halo, or the remapped index is still outside
            if bname == "wrap" and any(s < w // 2 for w, s in zip(widths, shp)):
                continue
            b = {"constant": A.constant(A.i64, -3), "function": Q.boundary_function(A.i64, len(shp))}.get(bname, bname)
            add("stencil_%s_%s_%s" % ("x".join(map(str, widths)), shp, bname),
                Q.stencil_weighted(A.i64, widths, b), [_rand(rng, A.i64, shp, -9, 9)], None)
    g = rng.uniform(0, 1, (37, 53)).astype(np.float32)
    add("jacobi_37x53", P.jacobi_step(), [g], None)
    add("stencil2_clamp_const", Q.stencil2_sum(A.f32, "clamp", A.constant(A.f32, 0.5)),
        [g, rng.uniform(0, 1, (40, 50)).astype(np.float32)], None)
    # stencil2 (Prelude/Stencil.hs): every boundary kind on either source, sources of different
    # extents (the result has their intersection), Int64 so that the comparison is exact
    s2 = lambda k: {"constant": A.constant(A.i64, 4), "function": Q.boundary_function(A.i64, 2)}.get(k, k)
    for b1, b2 in (("clamp", "wrap"), ("mirror", "clamp"), ("wrap", "mirror"), ("constant", "function"),
                   ("function", "constant"), ("wrap", "wrap"), ("mirror", "mirror")):
        for sh1, sh2 in (((5, 8), (7, 6)), ((70, 300), (64, 310)), ((2, 2), (2, 2))):
            add("stencil2_%s_%s_%s" % (b1, b2, sh1), Q.stencil2_sum(A.i64, s2(b1), s2(b2)),
                [_rand(rng, A.i64, sh1, -9, 9), _rand(rng, A.i64, sh2, -9, 9)], None)
    # ---- Transform (AST.hs:289-296): an index function and a value function in one node
    for shp in ((5, 7), (64, 300), (1, 1), (0, 4)):
        add("transform_transpose_affine_%s" % (shp,), Q.transform_transpose_affine(), [_rand(rng, A.i64, shp)], None)
    add("transform_gather_scale", Q.transform_gather_scale(),
        [rng.integers(0, 100, 257).astype(np.int64), _rand(rng, A.f32, (100,))], None)
    # ---- whole programs (Test/NoFib/Spectral: SMVM, RadixSort; Prelude/Filter.hs)
    for nrows, ncols in ((40, 30), (700, 500)):
        segd = rng.integers(0, 7, nrows).astype(np.int64)
        nnz = int(segd.sum())
        inds = rng.integers(0, ncols, nnz).astype(np.int64)
        add("smvm_i64_%d" % nrows, Q.smvm(A.i64),
            [segd, inds, _rand(rng, A.i64, (nnz,), -9, 9), _rand(rng, A.i64, (ncols,), -9, 9)], None)
        add("smvm_f32_%d" % nrows, Q.smvm(A.f32),
            [segd, inds, _rand(rng, A.f32, (nnz,)), _rand(rng, A.f32, (ncols,))], 1e-4 * 16 * 7)
    for n in (0, 1, 300, 5000):
        add("filter_positive_%d" % n, Q.filter_positive(), [_rand(rng, A.i64, (n,), -50, 50)], None)
    add("filter_none_pass", Q.filter_positive(), [-np.abs(_rand(rng, A.i64, (200,), -50, 50)) - 1], None)
    add("radix_4_passes", Q.radix_passes(4), [rng.integers(0, 16, 500).astype(np.int64)], None)
    add("radix_6_passes", Q.radix_passes(6), [rng.integers(0, 64, 3000).astype(np.int64)], None)
    # ---- segmented scans (Prelude.hs:958-1322): scan', permute, a flagged scan over a fused zip
    for shp, nseg in (((7, 900), 60), ((3, 6000), 25), ((2, 40), 0)):
        lens = rng.integers(0, max(2, 2 * shp[1] // max(1, nseg)), nseg).astype(np.int64)
        while lens.sum() > shp[1]:
            lens[int(np.argmax(lens))] //= 2
        m = _rand(rng, A.i64, shp, -20, 20)
        if nseg:     # the inclusive scans need a non-empty segment descriptor (Prelude.hs:1107-1110)
            add("scanl1seg_%s_%d" % (shp, nseg), Q.scan1_seg("l"), [m, lens], None)
            add("scanr1seg_%s_%d" % (shp, nseg), Q.scan1_seg("r"), [m, lens], None)
        add("scanlseg_%s_%d" % (shp, nseg), Q.scanl_seg(A.i64, 3), [m, lens], None)
    # ---- SIMD vector element types (Prelude/SIMD.hs:40-190): extract and inject for every base type
    #      and width, then vectors as the elements of scans, folds, permute, backpermute, stencil
    for k, ty in enumerate((A.i8, A.i16, A.i32, A.i64, A.u8, A.u16, A.u32, A.u64, A.f16, A.f32, A.f64)):
        for n in (2, 3, 4):
            xs = _rand(rng, ty, (157, n), -50, 50) if ty not in (A.f16, A.f32, A.f64) else _rand(rng, ty, (157, n))
            add("simd_extract_v%d_%s" % (n, ty), Q.vec_extract(n, ty, (k + n) % n), [xs], None)
            add("simd_inject_v%d_%s" % (n, ty), Q.vec_inject(n, ty), [xs[:150 - 7 * j, j].copy() for j in range(n)], None)
    add("simd_extract_v8_f16_rank2", Q.vec_extract(8, A.f16, 5, 2), [_rand(rng, A.f16, (9, 13, 8))], None)
    add("simd_extract_v16_i8", Q.vec_extract(16, A.i8, 11), [_rand(rng, A.i8, (300, 16), -100, 100)], None)
    add("simd_extract_empty", Q.vec_extract(3, A.i32, 2), [np.zeros((0, 3), np.int32)], None)
    for shp in ((1,), (300,), (5000,), (7, 900)):
        add("scan1_simd_v3i32_%s" % (shp,), Q.vec_scan(3, A.i32, "l", len(shp)), [_rand(rng, A.i32, shp + (3,), -50, 50)], None)
        add("scan1_simd_v2i64_r_%s" % (shp,), Q.vec_scan(2, A.i64, "r", len(shp)), [_rand(rng, A.i64, shp + (2,), -50, 50)], None)
    add("scan1_simd_v16i8", Q.vec_scan(16, A.i8), [_rand(rng, A.i8, (3000, 16), -100, 100)], None)
    add("fold_simd_v2i64", Q.vec_fold(2, A.i64), [_rand(rng, A.i64, (37, 1000, 2), -50, 50)], None)
    add("fold_simd_v3i16_rows", Q.vec_fold(3, A.i16), [_rand(rng, A.i16, (900, 7, 3), -50, 50)], None)
    add("permute_simd_v3i32", Q.vec_accumulate(3, A.i32, 17),
        [_rand(rng, A.i32, (2000, 3), -50, 50), rng.integers(0, 17, 2000).astype(np.int64)], None)
    add("simd_reverse_v3i16", Q.vec_reverse(3, A.i16), [_rand(rng, A.i16, (1001, 3), -50, 50)], None)
    add("stencil_simd_v2f32", Q.vec_stencil_1d(), [_rand(rng, A.f32, (777, 2))], None)
    # ---- Issue114: compensated summation over (value, error) pairs, a non-commutative fold1 / scanl1
    ef = [np.full(100, 1.01, np.float32), np.zeros(100, np.float32)]
    add("fold1_issue114", Q.issue114("fold1"), [ef], 1e-4 * 101)
    add("scan1_issue114", Q.issue114("scanl1"), [ef], 1e-4 * 101)
    # ---- Spectral/BlackScholes, Imaginary/SAXPY and SASUM (transcendental functions come from
    #      different libraries on the two sides: a few units in the last place)
    for ty, tol in ((A.f32, 2e-4), (A.f64, 1e-11)):
        psy = [rng.uniform(5, 30, 3000).astype(NPT[ty]), rng.uniform(1, 100, 3000).astype(NPT[ty]),
               rng.uniform(0.25, 10, 3000).astype(NPT[ty])]
        add("map_blackscholes_%s" % ty, Q.blackscholes(ty), [psy], tol)
        add("map_saxpy_%s" % ty, Q.saxpy(ty), [np.array(1.75, NPT[ty]), _rand(rng, ty, (2000,)), _rand(rng, ty, (1900,))], None)
        add("fold_sasum_%s" % ty, Q.sasum(ty), [_rand(rng, ty, (5000,))], 1e-4 * 4 * 5000 if ty == A.f32 else 1e-9)
    # ---- the benchmark programs at small size
    add("dotp_1000", P.dotp(), [_rand(rng, A.f32, (1000,)), _rand(rng, A.f32, (900,))], 1e-4 * 16 * 900)
    add("histogram_zipf", P.histogram(97), [rng.integers(0, 97, 3000).astype(np.int32)], None)
    add("map_affine", P.map_affine(), [_rand(rng, A.f32, (1234,))], None)
    return out


def gpu_only_programs():
    """Programs that only GPU tests run (larger inputs, forced kernel variants): compiled by
    the CPU suite too, so that their code objects travel in the kernel cache."""
    out = []
    for bname in ("clamp", "mirror", "wrap", "constant", "function"):
        for rank, widths_list in ((2, ([3, 3], [5, 3], [3, 5])), (3, ([3, 3, 3], [5, 3, 3], [3, 5, 7]))):
            b = {"constant": A.constant(A.i64, -3), "function": Q.boundary_function(A.i64, rank)}.get(bname, bname)
            for widths in widths_list:
                out.append(("stencil_%s_%s" % (widths, bname), Q.stencil_weighted(A.i64, widths, b)))
    for nb in (1 << 20, (1 << 21) + 12345, 1 << 22):
        out.append(("histogram_%d" % nb, P.histogram(nb)))
    out.append(("transpose_i32", Q.transpose(A.i32)))
    out.append(("transpose_i64", Q.transpose(A.i64)))
    return out

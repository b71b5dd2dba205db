"""Parity of the HIP backend with the oracle, through the C ABI, on a real MI355X.

Bar: bit-exact for every integer / index result and for Float32 code without a reduction
(map, stencil); Float32 reductions and scans within |gpu - ref| <= 1e-4 * sum |x_i| per
output element (the tolerance the benchmark definition states), written at each case.
"""
import numpy as np
import pytest

from accelerate_amd import hip
from accelerate_amd import ir as A
from accelerate_amd import programs as P
from accelerate_amd import workloads as W
from oracle import c as OC
from oracle import interp as O

from . import progs as Q
from .cases import golden_cases, parity_cases, same

pytestmark = pytest.mark.gpu

GOLDEN = golden_cases()
PARITY = parity_cases()


def test_native_library_is_what_runs(gpu_ctx):
    # the shared library is loaded and a device context exists: no eager / CPU path can answer
    assert hip.lib() is not None and gpu_ctx.mem_info()[0] > 100 << 30


@pytest.mark.parametrize("case", GOLDEN, ids=[c[0] for c in GOLDEN])
def test_reference_known_answers(gpu_ctx, case):
    _, prog, args, expected = case
    assert same(gpu_ctx.compile(prog)(*args), expected)


@pytest.mark.parametrize("case", PARITY, ids=[c[0] for c in PARITY])
def test_random_cases_match_oracle(gpu_ctx, case):
    _, prog, args, tol = case
    got = gpu_ctx.compile(prog)(*args)
    exp = O.run_n(prog.text(), *args)
    if tol is None:
        assert same(got, exp)
    else:
        assert same(got, exp, exact=False, atol=tol)


SCANS = [(c, g) for cs, g in ((GOLDEN, True), (PARITY, False)) for c in cs if "scan" in c[0] or "foldseg" in c[0]]


@pytest.mark.parametrize("tiles", ["large", "small", "rows"])
@pytest.mark.parametrize("case", SCANS, ids=[c[0][0] for c in SCANS])
def test_scans_with_either_tile_size(gpu_ctx, knobs, case, tiles):
    # rows this short take the small-tile kernel or, several rows per workgroup, the rows
    # kernel by default; every variant must agree with the reference's known answers and with
    # the oracle on every case ("rows" falls back to tiles where a row exceeds a tile)
    knobs("scan_tiles", {"large": 1, "small": 2, "rows": 3}[tiles])
    (_, prog, args, last), golden = case
    got = gpu_ctx.compile(prog)(*args)
    if golden:
        assert same(got, last)
    elif last is None:
        assert same(got, O.run_n(prog.text(), *args))
    else:
        assert same(got, O.run_n(prog.text(), *args), exact=False, atol=last)


FOLDS = [(c, g) for cs, g in ((GOLDEN, True), (PARITY, False)) for c in cs
         if c[0].startswith(("fold", "dotp", "mss", "issue228")) and "foldseg" not in c[0]]


@pytest.mark.parametrize("rows_kernel", ["0", "1", "2"])
@pytest.mark.parametrize("case", FOLDS, ids=[c[0][0] for c in FOLDS])
def test_folds_with_and_without_the_rows_kernel(gpu_ctx, knobs, case, rows_kernel):
    # short rows are reduced several per workgroup (1), or by a few lanes of a wave each (2); all
    # paths must give the same answers
    knobs("fold_rows", int(rows_kernel))
    (_, prog, args, last), golden = case
    got = gpu_ctx.compile(prog)(*args)
    if golden:
        assert same(got, last)
    elif last is None:
        assert same(got, O.run_n(prog.text(), *args))
    else:
        assert same(got, O.run_n(prog.text(), *args), exact=False, atol=last)


def test_fold_over_several_launches(gpu_ctx, knobs):
    # more rows than one launch holds workgroups (2^24 at 256 threads) take several launches;
    # forced here at a small size: 1000 rows, 7 workgroups per launch, with and without rows that
    # are split over workgroups
    knobs("fold_max_blocks", 7)
    knobs("fold_rows", 0)
    rng = np.random.default_rng(78)
    for shp in [(1000, 33), (5, 100_000)]:
        x = rng.integers(-50, 50, shp).astype(np.int64)
        assert same(gpu_ctx.compile(P.fold_sum(A.i64, 2))(x), x.sum(axis=1))


def test_rows_reduced_by_a_few_lanes_each(gpu_ctx, knobs):
    # lengths around the powers of two that decide how many lanes a row gets, ragged last runs,
    # fewer rows than a wave holds, a seed, an operator on pairs of bits, a maximum
    knobs("fold_rows", 2)
    rng = np.random.default_rng(31)
    sums = gpu_ctx.compile(P.fold_sum(A.i32, 2, 7))
    maxs = gpu_ctx.compile(P.fold1_op(A.max_, A.i64, 2))
    for rows, n in [(1, 1), (3, 2), (1000, 3), (777, 4), (64, 5), (999, 17), (4096, 64), (100, 255), (100, 256), (100, 257),
                    (50, 1000), (33, 4095), (7, 10_001), (300_000, 12)]:
        x = rng.integers(-1000, 1000, (rows, n))
        assert np.array_equal(sums(x.astype(np.int32)), (7 + x.sum(axis=1)).astype(np.int32)), (rows, n)
        assert np.array_equal(maxs(x.astype(np.int64)), x.max(axis=1)), (rows, n)
    x = rng.random((5000, 300), dtype=np.float32)
    got = gpu_ctx.compile(P.fold_sum(A.f32, 2))(x)
    assert np.allclose(got, x.astype(np.float64).sum(axis=1), rtol=1e-5)
    x3 = rng.integers(-5, 5, (20, 30, 40)).astype(np.int64)
    assert np.array_equal(gpu_ctx.compile(P.fold_sum(A.i64, 3))(x3), x3.sum(axis=2))


@pytest.mark.parametrize("rows_kernel", [2, -1])
def test_rows_reduced_by_a_few_lanes_each_in_order(gpu_ctx, knobs, rows_kernel):
    # operators that are not commutative: "the last value that is not zero" and, on pairs, "the first
    # of the first and the second of the last" -- a lane then takes a stretch of its row, and any
    # stretch, run or lane joined out of order shows
    knobs("fold_rows", rows_kernel)
    rng = np.random.default_rng(32)
    I = A.i64
    last = A.lam([I, I], lambda p, q: A.cond(A.neq(I, q, A.constI(0)), q, p))
    lasts = gpu_ctx.compile(A.alam([A.tarray(2, I)], lambda xs: A.fold(last, A.constI(0), xs)))
    t2 = A.ttup(I, I)
    ends = gpu_ctx.compile(A.alam([A.tarray(2, t2)], lambda xs: A.fold(
        A.lam([t2, t2], lambda p, q: A.tup(A.untup(p)[0], A.untup(q)[1])), None, xs)))
    for rows, n in [(1, 1), (3, 2), (1000, 3), (64, 5), (999, 17), (4096, 64), (300, 127), (300, 128), (300, 129), (100, 255),
                    (100, 257), (50, 1000), (33, 4095), (7, 10_001), (300_000, 12), (70_000, 200)]:
        x = rng.integers(1, 1 << 40, (rows, n)).astype(np.int64)
        x[rng.random((rows, n)) < 0.7] = 0
        idx = np.where(x != 0, np.arange(n), -1).max(axis=1)
        want = np.where(idx >= 0, x[np.arange(rows), np.maximum(idx, 0)], 0)
        assert np.array_equal(lasts(x), want), (rows, n)
        y = rng.integers(-1000, 1000, (rows, n)).astype(np.int64)
        a, b = ends(gpu_ctx.to_device((x, y), A.tarray(2, t2)))
        assert np.array_equal(a, x[:, 0]) and np.array_equal(b, y[:, -1]), (rows, n)


@pytest.mark.parametrize("staged", [1, 0])
def test_long_rows_in_order(gpu_ctx, knobs, staged):
    # operators that are not commutative over chunks of 64 KiB and more: blocks of eight tiles are
    # turned over in LDS so that a lane combines a stretch in order; lengths around the block size
    # (1024 Int64), chunks that end in single tiles and ragged ones, several rows
    knobs("fold_staged", staged)
    rng = np.random.default_rng(33)
    I = A.i64
    last = A.lam([I, I], lambda p, q: A.cond(A.neq(I, q, A.constI(0)), q, p))
    t2 = A.ttup(I, I)
    ends = A.lam([t2, t2], lambda p, q: A.tup(A.untup(p)[0], A.untup(q)[1]))
    for rank, shape in [(1, (8192,)), (1, (32768,)), (1, (32769,)), (1, (100_003,)), (1, ((1 << 21) + 77,)), (2, (3, 40_000)),
                        (2, (2, 1 << 19))]:
        x = rng.integers(1, 1 << 40, shape).astype(np.int64)
        x[rng.random(shape) < 0.9] = 0
        n = shape[-1]
        idx = np.where(x != 0, np.arange(n), -1).max(axis=-1)
        want = np.where(idx >= 0, np.take_along_axis(x, np.maximum(idx, 0)[..., None], axis=-1)[..., 0], 0)
        got = gpu_ctx.compile(A.alam([A.tarray(rank, I)], lambda xs: A.fold(last, A.constI(0), xs)))(x)
        assert np.array_equal(got, want), shape
        y = rng.integers(-1000, 1000, shape).astype(np.int64)
        a, b = gpu_ctx.compile(A.alam([A.tarray(rank, t2)], lambda xs: A.fold(ends, None, xs)))(
            gpu_ctx.to_device((x, y), A.tarray(rank, t2)))
        assert np.array_equal(a, x[..., 0]) and np.array_equal(b, y[..., -1]), shape


@pytest.mark.parametrize("one_launch", [0, 1])
def test_single_row_with_and_without_the_second_launch(gpu_ctx, knobs, one_launch):
    # a single row cut into chunks: either a second launch combines the chunk results, or the
    # workgroup of the last chunk does, reading the others' results as tagged words; both in order
    # (the maximum segment sum's operator is not commutative), several calls in a row so that
    # words left by one call are met by the next, and at lengths where the last chunk is ragged
    knobs("fold_one_launch", one_launch)
    rng = np.random.default_rng(79)
    run = gpu_ctx.compile(Q.mss(A.Int, 1))
    total = gpu_ctx.compile(P.fold_sum(A.i64, 1, 7))
    for n in (2_000_001, 300_000, 5_000_017, 70_001):
        x = rng.integers(-50, 50, n).astype(np.int64)
        c = np.concatenate(([0], np.cumsum(x)))
        assert int(run(x)) == int((c - np.minimum.accumulate(c)).max()), n
        assert int(total(x)) == 7 + int(x.sum()), n
    a, b = W.uniform_f32(1 << 24, 11, 0.0, 1.0), W.uniform_f32(1 << 24, 12)
    got = float(gpu_ctx.compile(P.dotp())(a, b))
    ref = float(np.dot(a.astype(np.float64), b.astype(np.float64)))
    assert abs(got - ref) <= 1e-4 * float(np.sum(np.abs(a.astype(np.float64) * b)))


def test_rows_split_over_workgroups_are_combined_in_order(gpu_ctx):
    # rows long enough for several workgroups each, whose partial results a second launch
    # combines: a non-commutative operator (the maximum segment sum's) shows a partial out of
    # place; pinned by a numpy restatement
    rng = np.random.default_rng(77)
    for shp in [(3, 300_000), (1, 2_000_001), (17, 70_000)]:
        x = rng.integers(-50, 50, shp).astype(np.int64)
        run = gpu_ctx.compile(Q.mss(A.Int, 2))
        want = []
        for row in x:                      # Kadane's maximum segment sum, empty segment allowed
            c = np.concatenate(([0], np.cumsum(row)))
            want.append(int((c - np.minimum.accumulate(c)).max()))
        for _ in range(2):
            assert same(run(x), np.array(want, np.int64))
    y = rng.random((2, 1 << 20), dtype=np.float32)
    got = gpu_ctx.compile(P.fold_sum(A.f32, 2))(y)
    assert np.allclose(got, y.astype(np.float64).sum(axis=1), rtol=1e-5)


ELEMENTWISE = [(c, g) for cs, g in ((GOLDEN, True), (PARITY, False)) for c in cs
               if c[0].startswith(("map", "transpose", "gather", "identity", "issue185", "misc", "filter", "smvm",
                                   "radix", "fold", "dotp", "mss", "issue228"))
               and "foldseg" not in c[0]]


@pytest.mark.parametrize("case", ELEMENTWISE, ids=[c[0][0] for c in ELEMENTWISE])
def test_streaming_variants_of_map_and_fold(gpu_ctx, knobs, case):
    # launches that move far more than the last-level cache holds use kernels with
    # non-temporal accesses; forced here at every size, the answers must not change
    knobs("stream_bytes", 0)
    knobs("fold_rows", 0)
    (_, prog, args, last), golden = case
    got = gpu_ctx.compile(prog)(*args)
    if golden:
        assert same(got, last)
    elif last is None:
        assert same(got, O.run_n(prog.text(), *args))
    else:
        assert same(got, O.run_n(prog.text(), *args), exact=False, atol=last)


# ---- the five benchmark configurations at the size the oracle's C loops handle in seconds ----

def test_dotp_2pow24(gpu_ctx):
    n = 1 << 24
    x, y = W.uniform_f32(n, 1), W.uniform_f32(n, 2)
    got = gpu_ctx.compile(P.dotp())(x, y)
    exact = np.dot(x.astype(np.float64), y.astype(np.float64))
    bound = 1e-4 * np.sum(np.abs(x.astype(np.float64) * y))    # 1e-4 * sum |x_i * y_i|
    assert abs(float(got) - exact) <= bound
    assert abs(float(OC.dotp_f32(x, y)) - exact) <= bound      # the sequential reference meets the same bound


def test_scanl1_int64_2pow28_bit_exact(gpu_ctx):
    n = 1 << 28
    x = W.uniform_int(n, 3)
    got = gpu_ctx.compile(P.scanl1_sum(A.i64))(x)
    ref = OC.scanl1_i64(x)
    assert np.array_equal(got, ref)
    # size-independent properties: first difference restores the input, last element is the total
    assert got[0] == x[0] and np.array_equal(np.diff(got), x[1:]) and got[-1] == x.sum()


def test_scanl1_float32_2pow28_within_tolerance(gpu_ctx):
    n = 1 << 28
    x = W.uniform_f32(n, 4, 0.0, 1.0)
    got = gpu_ctx.compile(P.scanl1_sum(A.f32))(x)
    exact = np.cumsum(x, dtype=np.float64)                      # = sum_{k<=i} |x_k| since x >= 0
    assert np.all(np.abs(got - exact) <= 1e-4 * exact + 1e-30)
    assert np.all(np.diff(got[:: 1 << 16]) >= 0)                # monotone for non-negative input


def test_foldseg_2pow27_bit_exact(gpu_ctx):
    nseg, total = 1 << 20, 1 << 27
    lens, vals = W.segment_lengths(nseg, total, 5), W.uniform_int(total, 6, dtype=np.int32)
    got = gpu_ctx.compile(P.foldseg_sum())(vals, lens)
    assert np.array_equal(got, OC.foldseg_i32(vals, lens))
    assert got.sum(dtype=np.int64) & 0xFFFFFFFF == int(vals.sum(dtype=np.int64)) & 0xFFFFFFFF   # sum of sums
    assert np.all(got[lens == 0] == 0)


@pytest.mark.parametrize("one_launch", [1, 0], ids=["ends completed in the launch", "ends completed by a second launch"])
@pytest.mark.parametrize("shape", ["one giant segment", "giants and dwarfs", "runs of empty segments",
                                   "empty segments at the end", "single elements"])
def test_foldseg_segment_shapes_bit_exact(gpu_ctx, knobs, shape, one_launch):
    # segments that span hundreds of tiles (the carries of many tiles are chained), tiles
    # with far more boundaries than elements (runs of empty segments), and length-1 segments;
    # the ends that reach across tile borders completed by the workgroups behind the tiles, or
    # by the same code as a launch of its own
    knobs("foldseg_one_launch", one_launch)
    rng = np.random.default_rng(77)
    total = 1 << 23
    if shape == "one giant segment":
        lens = np.array([total], np.int32)
    elif shape == "giants and dwarfs":
        lens = np.array([5, 3_000_000, 0, 1, total - 3_000_006 - 700_001, 700_001], np.int32)
    elif shape == "runs of empty segments":
        total = 1 << 16
        lens = np.concatenate([[40000], np.zeros(50_000, np.int32), [20000], np.zeros(70_000, np.int32),
                               [total - 60000 - 7, 7], np.zeros(3, np.int32)]).astype(np.int32)
    elif shape == "empty segments at the end":
        total = 1 << 18
        lens = np.concatenate([np.full(total // 64, 64, np.int32), np.zeros(100_000, np.int32)])
    else:
        total = 1 << 20
        lens = np.ones(total, np.int32)
    vals = rng.integers(-1000, 1000, total).astype(np.int32)
    got = gpu_ctx.compile(P.foldseg_sum())(vals, lens)
    assert np.array_equal(got, OC.foldseg_i32(vals, lens))


def test_foldseg_calls_in_a_row_do_not_see_each_others_carries(gpu_ctx):
    # the carries of the tiles travel as tagged words in memory that the next call uses again:
    # a long call, a shorter one whose tiles end elsewhere, the long one again
    run = gpu_ctx.compile(P.foldseg_sum())
    rng = np.random.default_rng(5)
    cases = []
    for total, mean in ((1 << 22, 3000), (1 << 20, 70000), (1 << 22, 9000)):
        lens = rng.integers(0, 2 * mean, total // mean).astype(np.int64)
        lens = lens[np.cumsum(lens) <= total]
        lens = np.append(lens, total - lens.sum()).astype(np.int32)
        cases.append((rng.integers(-1000, 1000, total).astype(np.int32), lens))
    for vals, lens in cases + cases[::-1]:
        assert np.array_equal(run(vals, lens), OC.foldseg_i32(vals, lens))


def test_histogram_2pow26_bit_exact(gpu_ctx):
    n, nbins = 1 << 26, 1 << 16
    keys = W.zipf_keys(n, nbins, 7)
    got = gpu_ctx.compile(P.histogram(nbins))(keys)
    assert np.array_equal(got, OC.histogram_i32(keys, nbins))
    assert got.sum(dtype=np.int64) == n and np.array_equal(got, np.bincount(keys, minlength=nbins))


def test_map_over_several_launches(gpu_ctx, knobs):
    # index spaces of 2^32 threads and more are covered by several launches of the map skeleton;
    # here the limit is lowered to 3 workgroups so that small arrays take that path: a plain map,
    # an indexed generate of rank 3 and a directly evaluated stencil (XCD-contiguous numbering)
    knobs("map_max_blocks", 3)
    knobs("stencil_no2d", 1)
    rng = np.random.default_rng(5)
    x = rng.standard_normal(50001).astype(np.float32)
    assert np.array_equal(gpu_ctx.compile(P.map_affine())(x), x * np.float32(2) + np.float32(1))
    cube = rng.standard_normal((7, 33, 65)).astype(np.float32)
    prog = Q.indexed(3)
    assert same(gpu_ctx.compile(prog)(cube), O.run_n(prog.text(), cube))
    g = rng.uniform(0, 1, (67, 131)).astype(np.float32)
    assert same(gpu_ctx.compile(P.jacobi_step())(g), OC.jacobi_f32(g, 1))


def test_arrays_of_more_than_2p32_elements(gpu_ctx):
    # linear indices, grids and tile counts beyond 32 bits: a fold over a delayed source of
    # 2^32 + 5 elements (closed form), a manifest map over as many bytes read back at its far
    # end, and scanl1 over 2^31 + 3 Int32 ones, whose last prefixes wrap around
    big, n = (1 << 32) + 5, (1 << 31) + 3
    fold, far_end, scan_end = Q.long_array_programs(big, n)
    assert int(gpu_ctx.compile(fold)()) == Q.long_fold_expected(big)
    assert np.array_equal(gpu_ctx.compile(far_end)(), ((np.arange(big - 8, big) & 255) + 1).astype(np.uint8))
    assert np.array_equal(gpu_ctx.compile(scan_end)(), np.arange(n - 5, n + 1, dtype=np.int64).astype(np.int32))
    gpu_ctx.purge()


TILE_EDGES = sorted({t * k + d for t in (4096, 8192, 12288, 16384, 24576, 49152) for k in (1, 2, 5) for d in (-1, 0, 1)})


@pytest.mark.parametrize("tiles", ["large", "small"])
@pytest.mark.parametrize("ty", [A.i32, A.i64])
def test_scans_and_folds_at_tile_borders(gpu_ctx, knobs, ty, tiles):
    # lengths one short of, equal to and one beyond multiples of every tile size the scans use,
    # through both tile variants: left, right and exclusive scans and the fold, against numpy
    knobs("scan_tiles", {"large": 1, "small": 2, "rows": 3}[tiles])
    dt = np.int32 if ty == A.i32 else np.int64
    rng = np.random.default_rng(77)
    progs = {"scanl1": gpu_ctx.compile(P.scanl1_sum(ty)), "scanl'": gpu_ctx.compile(P.scan_prime_sum("l", ty, 1, 3)),
             "scanr": gpu_ctx.compile(P.scan_sum("r", ty, 1, 3)), "fold": gpu_ctx.compile(P.fold_sum(ty, 1, 3))}
    for n in TILE_EDGES:
        x = rng.integers(-1000, 1000, n).astype(dt)
        inc = np.cumsum(x, dtype=dt)
        assert np.array_equal(progs["scanl1"](x), inc), n
        body, total = progs["scanl'"](x)
        assert np.array_equal(body, np.concatenate([[3], 3 + inc[:-1]]).astype(dt)) and total == dt(3) + inc[-1], n
        rinc = np.cumsum(x[::-1], dtype=dt)[::-1]
        assert np.array_equal(progs["scanr"](x), np.concatenate([rinc + dt(3), [3]]).astype(dt)), n
        assert progs["fold"](x) == dt(3) + inc[-1], n


@pytest.mark.parametrize("tiles", ["large", "small", "rows"])
def test_scan_whose_function_indexes_a_table_at_tile_borders(gpu_ctx, knobs, tiles):
    # composition of finite-state transitions: the combination function reads tbl[a * k + b].  The
    # kernels apply it to every lane of a tile, also to lanes past the end of a row, so those lanes
    # must hold values of the array: anything else indexes outside the table.  Lengths around
    # the multiples of every tile size, against a sequential fold of the same table.
    knobs("scan_tiles", {"large": 1, "small": 2, "rows": 3}[tiles])
    k = 7
    rng = np.random.default_rng(123)
    tbl = rng.integers(0, k, k * k).astype(np.int64)
    # make the table's operation associative: composition of functions on k states, elements
    # are function numbers in a closed set; the simplest closed set is a cyclic group
    tbl = np.array([(a + b) % k for a in range(k) for b in range(k)], np.int64)
    runs = {(d, kind): gpu_ctx.compile(Q.table_scan(k, d, kind)) for d in "lr" for kind in ("scan1", "scan")}
    edges = TILE_EDGES if tiles != "rows" else [1, 2, 63, 64, 65, 1000, 2047, 2048, 4095, 4096]
    for n in edges:
        x = rng.integers(0, k, n).astype(np.int64)
        inc = np.cumsum(x) % k
        rinc = (np.cumsum(x[::-1]) % k)[::-1]
        assert np.array_equal(runs[("l", "scan1")](tbl, x), inc), n
        assert np.array_equal(runs[("r", "scan1")](tbl, x), rinc), n
        assert np.array_equal(runs[("l", "scan")](tbl, x), np.concatenate([[0], inc])), n
        assert np.array_equal(runs[("r", "scan")](tbl, x), np.concatenate([rinc, [0]])), n


def test_many_short_rows_of_a_table_scan(gpu_ctx):
    # the rows kernel: several whole rows per workgroup, the last workgroup ragged
    k = 5
    tbl = np.array([(a + b) % k for a in range(k) for b in range(k)], np.int64)
    rng = np.random.default_rng(5)
    V1, V2 = A.tarray(1, A.Int), A.tarray(2, A.Int)
    prog = A.alam([V1, V2], lambda t, xs: A.scan("l", A.lam([A.Int, A.Int], lambda a, b: A.index(
        t, A.sh(A.add(A.Int, A.mul(A.Int, a, A.constI(k)), b)))), None, xs))
    run = gpu_ctx.compile(prog)
    for shape in ((1001, 7), (333, 100), (50, 1500), (3, 4097)):
        x = rng.integers(0, k, shape).astype(np.int64)
        assert np.array_equal(run(tbl, x), np.cumsum(x, axis=1) % k), shape


@pytest.mark.parametrize("nbins", [1 << 20, (1 << 21) + 12345, 1 << 22])
def test_histogram_over_many_lds_fuls(gpu_ctx, knobs, nbins):
    # destinations of up to 128 LDS-fuls are still combined in workgroup-private copies, one
    # range of the destination per pass; against numpy and against the plain global atomics
    keys = W.zipf_keys(1 << 22, nbins, 5)
    ref = np.bincount(keys, minlength=nbins)
    run = gpu_ctx.compile(P.histogram(nbins))
    assert np.array_equal(run(keys), ref)
    knobs("permute_parts", 0)
    assert np.array_equal(run(keys), ref)


def test_jacobi_8192_bit_equal(gpu_ctx):
    g = W.uniform_f32(8192 * 8192, 8, 0.0, 1.0).reshape(8192, 8192)
    step = gpu_ctx.compile(P.jacobi_step())
    d = gpu_ctx.to_device(g, A.tarray(2, A.f32))
    for _ in range(3):
        d = step.execute(d)
    got = d.to_host()
    assert np.array_equal(got, OC.jacobi_f32(g, 3))             # no reduction, no contraction: bit-equal
    assert got.min() >= g.min() and got.max() <= g.max()        # averaging never leaves the input's range


def test_jacobi_8192_100_iterations_bit_equal(gpu_ctx):
    # the stencil configuration at its full size: 100 sweeps over 8192 x 8192, every cell compared
    g = W.uniform_f32(8192 * 8192, 8, 0.0, 1.0).reshape(8192, 8192)
    step = gpu_ctx.compile(P.jacobi_step())
    d = gpu_ctx.to_device(g, A.tarray(2, A.f32))
    for _ in range(100):
        d = step.execute(d)
    got = d.to_host()
    assert np.array_equal(got, OC.jacobi_f32(g, 100))


def test_jacobi_8192_100_iterations_under_awhile_bit_equal(gpu_ctx):
    # the same configuration driven by awhile instead of repeated run1 (the configuration allows
    # either): the loop state is (grid, counter), the counter is followed on the host
    from .runtime_cases import jacobi_awhile
    g = W.uniform_f32(8192 * 8192, 8, 0.0, 1.0).reshape(8192, 8192)
    run = gpu_ctx.compile(jacobi_awhile(100))
    got = run.execute(gpu_ctx.to_device(g, A.tarray(2, A.f32))).to_host()
    assert np.array_equal(got, OC.jacobi_f32(g, 100))


def test_jacobi_100_iterations_small_grid_bit_equal(gpu_ctx):
    g = W.uniform_f32(96 * 160, 9, 0.0, 1.0).reshape(96, 160)
    step = gpu_ctx.compile(P.jacobi_step())
    d = gpu_ctx.to_device(g, A.tarray(2, A.f32))
    for _ in range(100):
        d = step.execute(d)
    assert np.array_equal(d.to_host(), OC.jacobi_f32(g, 100))


# ---- error conventions (Error.hs:33-62) -------------------------------------------------------

@pytest.mark.parametrize("chain", [2, 3, 7])
@pytest.mark.parametrize("bname", ["clamp", "mirror", "wrap", "constant", "function"])
def test_stencil_tile_chains_match_oracle(gpu_ctx, knobs, bname, chain):
    # a workgroup that walks down several tiles of a column (forced here; by default only
    # large arrays do that), on extents that leave ragged tiles at the right and bottom edge
    knobs("stencil_chain", chain)
    rng = np.random.default_rng(1000 + chain)
    b = {"constant": A.constant(A.i64, -3), "function": Q.boundary_function(A.i64, 2)}.get(bname, bname)
    for widths, shp in [([3, 3], (150, 70)), ([5, 3], (97, 130)), ([3, 5], (33, 64))]:
        prog = Q.stencil_weighted(A.i64, widths, b)
        x = rng.integers(-9, 10, shp).astype(np.int64)
        assert same(gpu_ctx.compile(prog)(x), O.run_n(prog.text(), x))


_ORACLE_3D = {}


@pytest.mark.parametrize("chain", [1, 3, 32])
@pytest.mark.parametrize("bname", ["clamp", "mirror", "wrap", "constant", "function"])
def test_stencil3d_plane_ring_matches_oracle(gpu_ctx, knobs, bname, chain):
    # rank 3: columns that march along z over a ring of planes in LDS; chains shorter than,
    # equal to and longer than the array, ragged columns at the y and x edges
    knobs("stencil_chain", chain)
    b = {"constant": A.constant(A.i64, -3), "function": Q.boundary_function(A.i64, 3)}.get(bname, bname)
    for n, (widths, shp) in enumerate([([3, 3, 3], (7, 11, 140)), ([5, 3, 3], (6, 8, 128)), ([3, 5, 7], (4, 19, 30))]):
        prog = Q.stencil_weighted(A.i64, widths, b)
        x = np.random.default_rng(2000 + n).integers(-9, 10, shp).astype(np.int64)
        if (bname, n) not in _ORACLE_3D:     # the same for every chain length
            _ORACLE_3D[(bname, n)] = O.run_n(prog.text(), x)
        assert same(gpu_ctx.compile(prog)(x), _ORACLE_3D[(bname, n)])


def test_stencil2d_direct_evaluation_matches_oracle():
    # the same direct evaluation forced for rank 2: rows long enough for threads whose results
    # and taps all lie inside a row (evaluated without tests) next to threads at the borders
    ctx = hip.Context(0)
    ctx.set_knob("stencil_no2d", 1)
    rng = np.random.default_rng(32)
    for bname in ("clamp", "mirror", "wrap", "constant", "function"):
        for ty, widths in ((A.i64, [3, 5]), (A.i32, [5, 3])):
            b = {"constant": A.constant(ty, -3), "function": Q.boundary_function(ty, 2)}.get(bname, bname)
            prog = Q.stencil_weighted(ty, widths, b)
            x = rng.integers(-9, 10, (9, 70)).astype(np.int64 if ty == A.i64 else np.int32)
            assert same(ctx.compile(prog)(x), O.run_n(prog.text(), x))
    ctx.close()


def test_stencil3d_direct_evaluation_matches_oracle():
    # the direct (one thread per result) evaluation that ranks other than 2 and 3 use, forced
    # here for rank 3
    ctx = hip.Context(0)
    ctx.set_knob("stencil_no3d", 1)
    rng = np.random.default_rng(31)
    for bname in ("clamp", "wrap", "constant"):
        b = {"constant": A.constant(A.i64, -3)}.get(bname, bname)
        prog = Q.stencil_weighted(A.i64, [3, 3, 3], b)
        x = rng.integers(-9, 10, (6, 7, 70)).astype(np.int64)
        assert same(ctx.compile(prog)(x), O.run_n(prog.text(), x))
    ctx.close()


@pytest.mark.parametrize("tiled", ["0", "1", None])
def test_transposes_with_and_without_tiles(gpu_ctx, knobs, tiled):
    # index-permuting producers go over 32 x 8V tiles of the result when it is large enough
    # (forced on and off here, ragged tiles included); left alone, the transposition of a matrix
    # moves through 64 x 64 tiles in LDS
    if tiled is not None:
        knobs("map_tiled", int(tiled))
    rng = np.random.default_rng(5)
    for ty, npt in ((A.i32, np.int32), (A.i64, np.int64), (A.f32, np.float32), (A.u8, np.uint8)):
        run = gpu_ctx.compile(Q.transpose(ty))
        for shp in [(33, 17), (100, 300), (64, 64), (5, 1000), (1, 1), (257, 3), (1000, 513), (4097, 130), (63, 65)]:
            x = rng.integers(0, 200, shp).astype(npt)
            assert np.array_equal(run(x), x.T)


@pytest.mark.parametrize("tiled", [None, "1", "0"])
def test_axis_permutations_of_rank_3_and_mirrored_transposes(gpu_ctx, knobs, tiled):
    # index-permuting producers whose source runs along another dimension than the result's innermost
    # one go through LDS tiles of the plane of the two (left alone), 32 x 8V tiles (1) or the linear
    # order (0); ragged extents, every pair of dimensions swapped, a transposition that also mirrors
    if tiled is not None:
        knobs("map_tiled", int(tiled))
    rng = np.random.default_rng(6)
    perms = {"inner two": (0, 2, 1), "outer two": (1, 0, 2), "first and last": (2, 1, 0), "rotate": (1, 2, 0)}
    for ty, npt in ((A.i32, np.int32), (A.i64, np.int64), (A.u8, np.uint8)):
        for shp in [(3, 70, 130), (65, 64, 63), (2, 300, 5), (40, 33, 257)]:
            x = rng.integers(0, 200, shp).astype(npt)
            for name, pm in perms.items():
                # result dimension d is source dimension pm[d]: result index ix reads source index src with src[pm[d]] = ix[d]
                inv = [pm.index(k) for k in range(3)]
                prog = Q.reindex(3, lambda dd, pm=pm: [dd()[pm[0]], dd()[pm[1]], dd()[pm[2]]],
                                 lambda ix, dd, inv=inv: [ix[inv[0]], ix[inv[1]], ix[inv[2]]], ty)
                assert np.array_equal(gpu_ctx.compile(prog)(x), x.transpose(pm)), (name, shp)
    # transposition with the rows mirrored: result (y, x) = source (x, h - 1 - y)
    m = rng.integers(0, 1000, (300, 517)).astype(np.int32)
    prog = Q.reindex(2, lambda dd: [dd()[1], dd()[0]],
                     lambda ix, dd: [ix[1], A.sub(A.Int, A.sub(A.Int, dd()[1], A.constI(1)), ix[0])], A.i32)
    assert np.array_equal(gpu_ctx.compile(prog)(m), m.T[::-1, :])


def test_more_than_2_pow_31_elements(gpu_ctx):
    # linear indices beyond 32 bits: a map, a fold and a scan over 2^31 + 1000 Word8 elements
    n = (1 << 31) + 1000
    x = np.arange(n, dtype=np.uint32).astype(np.uint8)
    x[-3:] = (7, 11, 13)
    dx = gpu_ctx.to_device(x, A.tarray(1, A.u8))
    inc = gpu_ctx.compile(A.alam([A.tarray(1, A.u8)], lambda xs: A.map_(
        A.u8, A.lam([A.u8], lambda v: A.add(A.u8, v, A.const(A.u8, 1))), xs)))
    got = inc.execute(dx).to_host()
    assert got.shape == (n,) and np.array_equal(got[-1000:], x[-1000:] + np.uint8(1)) and np.array_equal(got[:1000], x[:1000] + np.uint8(1))
    assert np.array_equal(got[1 << 31 : (1 << 31) + 8], x[1 << 31 : (1 << 31) + 8] + np.uint8(1))
    del got
    total = gpu_ctx.compile(P.fold_sum(A.u8, 1, 0)).execute(dx).to_host()
    assert int(total) == int(x.sum(dtype=np.uint64) & 0xFF)
    run = gpu_ctx.compile(P.scanl1_sum(A.u8)).execute(dx).to_host()
    assert run[-1] == total and np.array_equal(run[:4096], np.cumsum(x[:4096], dtype=np.uint8))
    assert np.array_equal(np.diff(run[-5000:]).astype(np.uint8), x[-4999:])


@pytest.mark.parametrize("kind,widths,shape", [("mirror", [3, 3], (1, 5)), ("mirror", [3, 3], (5, 1)), ("wrap", [9], (3,)),
                                               ("mirror", [9], (4,)), ("mirror", [3, 3, 3], (2, 1, 9)),
                                               ("wrap", [5, 5], (1, 11))])
def test_stencil_extent_too_short_for_its_boundary_is_a_bounds_error(gpu_ctx, kind, widths, shape):
    # Mirror on an extent <= halo and Wrap on an extent < halo leave the remapped index outside the
    # array; the reference reports it when it indexes the source (Shape.hs:98-106), so does the
    # oracle, and here the host refuses the launch
    prog = Q.stencil_weighted(A.i64, widths, kind)
    x = np.ones(shape, np.int64)
    with pytest.raises(O.OracleError, match="index out of bounds"):
        O.run_n(prog.text(), x)
    launches = gpu_ctx.stat("launches")
    with pytest.raises(hip.AccError, match="index out of bounds") as e:
        gpu_ctx.compile(prog)(x)
    assert e.value.code == 4 and gpu_ctx.stat("launches") == launches
    # one element more (Mirror) is enough
    ok = tuple(max(s, w // 2 + (1 if kind == "mirror" else 0)) for s, w in zip(shape, widths))
    y = np.arange(int(np.prod(ok)), dtype=np.int64).reshape(ok)
    assert same(gpu_ctx.compile(prog)(y), O.run_n(prog.text(), y))


def test_lookback_wait_is_bounded_and_reported(gpu_ctx, knobs):
    # Fault injection from the host: the launch is told a ticket count that lags the device's by
    # 3, so its tiles take numbers 3 too high -- the first ones wait for predecessors that never
    # run, the last ones fall outside the launch.  With a poll limit of 50 every workgroup still
    # finishes within microseconds; the condition is raised by the next wait on the stream and
    # the context stays usable.
    x = W.uniform_int(400_000, 3)
    run = gpu_ctx.compile(P.scanl1_sum(A.i64))
    assert np.array_equal(run(x), np.cumsum(x))
    knobs("scan_test_skew", 3)
    knobs("scan_spin_limit", 50)
    res = run.execute(gpu_ctx.to_device(x, A.tarray(1, A.i64)))
    with pytest.raises(hip.AccError, match="gave up waiting"):
        gpu_ctx.sync()
    res.release()
    knobs("scan_test_skew", 0)
    knobs("scan_spin_limit", 1 << 22)
    assert np.array_equal(run(x), np.cumsum(x))


def test_fold1_of_empty_is_a_bounds_error(gpu_ctx):
    with pytest.raises(hip.AccError) as e:
        gpu_ctx.compile(P.fold1_op(A.add, A.i32, 2))(np.zeros((3, 0), np.int32))
    assert e.value.code == 4 and "empty array" in str(e.value)


def test_empty_segment_descriptor_is_a_bounds_error(gpu_ctx):
    prog = A.alam([A.tarray(1, A.i32), A.tarray(1, A.i32)], lambda v, offs: A.foldseg(
        A.i32, Q.binop(A.add, A.i32), A.const(A.i32, 0), v, offs))
    with pytest.raises(hip.AccError) as e:
        gpu_ctx.compile(prog)(np.zeros(3, np.int32), np.zeros(0, np.int32))
    assert e.value.code == 4


def test_wrong_argument_type_is_rejected(gpu_ctx):
    run = gpu_ctx.compile(P.fold_sum(A.i32, 2, 0))
    wrong = gpu_ctx.to_device(np.zeros((2, 2), np.float32), A.tarray(2, A.f32))
    with pytest.raises(hip.AccError):
        run.execute(wrong)


def test_separable_blur_of_the_stencil_documentation(gpu_ctx):
    # Language.hs:912-930: a 5x5 Gaussian blur as two passes whose stencils have rows of different
    # widths -- Stencil5x1 = (Stencil3, Stencil5, Stencil3) reads only its middle row, Stencil1x5 =
    # five Stencil3 rows only their middle elements -- under clamp, and under mirror and wrap
    ty = A.f32
    kern = [0.06136, 0.24477, 0.38774, 0.24477, 0.06136]

    def conv(ts):
        acc = A.mul(ty, A.const(ty, kern[0]), ts[0])
        for w, t in zip(kern[1:], ts[1:]):
            acc = A.add(ty, acc, A.mul(ty, A.const(ty, w), t))
        return acc

    def blur5x1(b):
        sr = A.stup(A.sunit(3, ty), A.sunit(5, ty), A.sunit(3, ty))
        return A.alam([A.tarray(2, ty)], lambda g: A.stencil(
            sr, ty, A.lam([A.stencil_type(sr)], lambda st: conv(A.untup(A.untup(st)[1]))), b, g))

    def blur1x5(b):
        sr = A.stup(*[A.sunit(3, ty) for _ in range(5)])
        return A.alam([A.tarray(2, ty)], lambda g: A.stencil(
            sr, ty, A.lam([A.stencil_type(sr)], lambda st: conv([A.untup(r)[1] for r in A.untup(st)])), b, g))

    rng = np.random.default_rng(44)
    for shape in ((7, 9), (300, 517), (3, 40), (40, 3)):
        x = rng.random(shape, dtype=np.float32)
        for b in (A.clamp, A.mirror, A.wrap):
            for prog in (blur5x1(b), blur1x5(b)):
                assert same(gpu_ctx.compile(prog)(x), O.run_n(prog.text(), x)), (shape, b)
    # blur = stencil (convolve5x1 gaussian) clamp . stencil (convolve1x5 gaussian) clamp
    both = A.alam([A.tarray(2, ty)], lambda g: A.apply(blur5x1(A.clamp), A.apply(blur1x5(A.clamp), g)))
    x = rng.random((64, 70), dtype=np.float32)
    assert same(gpu_ctx.compile(both)(x), O.run_n(both.text(), x))

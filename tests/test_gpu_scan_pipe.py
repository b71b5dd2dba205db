"""The pipelined scan kernel (persistent workgroups, direct global -> LDS loads; scans over long
rows of a plain array with elements of 4 or 8 bytes, Interpreter.hs:427-474), forced onto every
case through the `scan_tiles` knob and compared with numpy and with the other tile variants.
A tile of it holds 1024 lanes x 128 bytes of 8-byte elements (16384 of them) or x 112 bytes of 4-byte
elements (28672)."""
import numpy as np
import pytest

from accelerate_amd import hip, ir as A, programs as P, workloads as W

from . import progs as Q

pytestmark = pytest.mark.gpu

TYPES = [(A.i32, np.int32, 28672), (A.i64, np.int64, 16384), (A.f32, np.float32, 28672), (A.f64, np.float64, 16384),
         (A.u32, np.uint32, 28672)]


def _lengths(tile):
    # one tile, whole numbers of tiles, one short of and one beyond them, a ragged many-tile row
    return [tile, 3 * tile, 3 * tile + 1, 5 * tile - 1, 40 * tile + 12345, 300 * tile]


def _close(got, want, npty):
    if np.dtype(npty).kind in "iu":
        return np.array_equal(got, want)
    # floating sums regroup: the configuration's bound, 1e-4 * sum |x_i|, is far wider than this
    return np.allclose(got, want, rtol=1e-5, atol=1e-5 * float(np.abs(want).max() + 1))


@pytest.mark.parametrize("ty,npty,tile", TYPES, ids=[t[0] for t in TYPES])
def test_left_scans_of_every_kind(gpu_ctx, knobs, ty, npty, tile):
    knobs("scan_tiles", 4)
    rng = np.random.default_rng(7)
    wide = np.float64 if np.dtype(npty).kind == "f" else npty
    runs = (gpu_ctx.compile(P.scanl1_sum(ty)), gpu_ctx.compile(P.scan_sum("l", ty, 1, 5)),
            gpu_ctx.compile(P.scan_prime_sum("l", ty, 1, 3)))
    for n in _lengths(tile):
        lo = 0 if np.dtype(npty).kind == "u" else -1000
        x = rng.integers(lo, 1000, n).astype(npty)
        inc = np.cumsum(x.astype(wide), dtype=wide)
        dx = gpu_ctx.to_device(x, A.tarray(1, ty))
        assert _close(runs[0].execute(dx).to_host(), inc.astype(npty), npty), ("scanl1", n)
        assert _close(runs[1].execute(dx).to_host(), np.concatenate([[5], 5 + inc]).astype(npty), npty), ("scanl", n)
        body, total = [p.to_host() for p in runs[2].execute(dx).parts()]
        assert _close(body, np.concatenate([[3], 3 + inc[:-1]]).astype(npty), npty), ("scanl'", n)
        assert _close(total, np.array(3 + inc[-1]).astype(npty), npty), ("scanl' total", n)


@pytest.mark.parametrize("ty,npty,tile", TYPES, ids=[t[0] for t in TYPES])
def test_right_scans_of_every_kind(gpu_ctx, knobs, ty, npty, tile):
    # a right scan walks over the row's mirror image; lengths that are not a multiple of 16 bytes
    # (the last two) take the other kernel, and must give the same
    knobs("scan_tiles", 4)
    rng = np.random.default_rng(8)
    wide = np.float64 if np.dtype(npty).kind == "f" else npty
    runs = (gpu_ctx.compile(P.scan1_sum("r", ty)), gpu_ctx.compile(P.scan_sum("r", ty, 1, 5)),
            gpu_ctx.compile(P.scan_prime_sum("r", ty, 1, 3)))
    for n in [tile, 3 * tile, 3 * tile + 4, 5 * tile - 4, 40 * tile + 12344, 300 * tile, 7 * tile + 1, 9 * tile - 3]:
        lo = 0 if np.dtype(npty).kind == "u" else -1000
        x = rng.integers(lo, 1000, n).astype(npty)
        inc = np.cumsum(x[::-1].astype(wide), dtype=wide)[::-1]      # inc[i] = x[i] + .. + x[n-1]
        dx = gpu_ctx.to_device(x, A.tarray(1, ty))
        assert _close(runs[0].execute(dx).to_host(), inc.astype(npty), npty), ("scanr1", n)
        assert _close(runs[1].execute(dx).to_host(), np.concatenate([5 + inc, [5]]).astype(npty), npty), ("scanr", n)
        body, total = [p.to_host() for p in runs[2].execute(dx).parts()]
        assert _close(body, np.concatenate([3 + inc[1:], [3]]).astype(npty), npty), ("scanr'", n)
        assert _close(total, np.array(3 + inc[0]).astype(npty), npty), ("scanr' total", n)


def test_right_scan_of_several_rows_with_an_operator_that_is_not_commutative(gpu_ctx, knobs):
    # a (+) b = a if a /= 0 else b: associative, not commutative; scanr1 gives every position the
    # nearest non-zero value at or to the right of it.  Rows of a whole number of 16 bytes.
    knobs("scan_tiles", 4)
    rows, n = 3, 16384 * 17 + 6
    rng = np.random.default_rng(3)
    x = rng.integers(1, 1 << 40, (rows, n)).astype(np.int64)
    x[rng.random((rows, n)) < 0.9995] = 0        # long stretches of zeros: values travel across many tiles
    f = A.lam([A.Int, A.Int], lambda a, b: A.cond(A.neq(A.Int, a, A.constI(0)), a, b))
    prog = A.alam([A.tarray(2, A.Int)], lambda xs: A.scan("r", f, None, xs))
    at = np.where(x != 0, np.arange(n)[None, :], n)
    nxt = np.minimum.accumulate(at[:, ::-1], axis=1)[:, ::-1]
    want = np.where(nxt < n, np.take_along_axis(x, np.minimum(nxt, n - 1), axis=1), 0)
    run = gpu_ctx.compile(prog)
    for tiles in (4, 1):
        knobs("scan_tiles", tiles)
        assert np.array_equal(run(x), want), tiles


def _scan_of_fused(ty, g, direction="l", seed=None, prime=False, extra=None):
    """scan (+) over a producer fused into it: \\i -> g (xs ! i), optionally reading a second array too"""
    sh1 = A.tshape(1)
    args = [A.tarray(1, ty)] + ([A.tarray(1, ty)] if extra else [])

    def body(a, *more):
        at_ix = lambda ix: g(A.index(a, A.vexp(ix)), *[A.index(m, A.vexp(ix)) for m in more])
        at_lin = lambda i: g(A.linearindex(a, i), *[A.linearindex(m, i) for m in more])
        src = A.delayed(A.tarray(1, ty), A.shape(a), A.lam([sh1], at_ix), A.lam([A.Int], at_lin))
        z = None if seed is None else A.const(ty, seed)
        return (A.scan_ if prime else A.scan)(direction, P._binop(A.add, ty), z, src)

    return A.alam(args, body)


def test_producers_fused_into_the_scan(gpu_ctx, knobs):
    # scanl f z (map g xs): a function of one array's element at the scan's own position rides
    # along in the pipelined kernel (applied to what arrives in LDS); one that reads two arrays
    # at that position keeps the other kernels.  Both give what numpy gives, in both directions.
    knobs("scan_tiles", 4)
    rng = np.random.default_rng(17)
    twice_plus = lambda v: A.add(A.i64, A.mul(A.i64, v, A.const(A.i64, 2)), A.const(A.i64, 1))
    for n in (16384 * 3, 16384 * 40 + 8, 16384 * 300):
        x = rng.integers(-1000, 1000, n).astype(np.int64)
        y = 2 * x + 1
        assert np.array_equal(gpu_ctx.compile(_scan_of_fused(A.i64, twice_plus))(x), np.cumsum(y)), n
        assert np.array_equal(gpu_ctx.compile(_scan_of_fused(A.i64, twice_plus, "r", 5))(x),
                              np.concatenate([5 + np.cumsum(y[::-1])[::-1], [5]])), n
        body, total = gpu_ctx.compile(_scan_of_fused(A.i64, twice_plus, "l", 3, True))(x)
        inc = 3 + np.cumsum(y)
        assert np.array_equal(body, np.concatenate([[3], inc[:-1]])) and total == inc[-1], n
        w = rng.integers(-1000, 1000, n).astype(np.int64)
        both = _scan_of_fused(A.i64, lambda v, u: A.add(A.i64, v, u), extra=True)
        assert np.array_equal(gpu_ctx.compile(both)(x, w), np.cumsum(x + w)), n
    # the element's type changes with the function (Int32 -> Float32: same size, so it still rides along)
    xi = rng.integers(0, 2, 28672 * 20).astype(np.int32)
    conv = A.alam([A.tarray(1, A.i32)], lambda a: A.scan("l", P._binop(A.add, A.f32), None, A.delayed(
        A.tarray(1, A.f32), A.shape(a), A.lam([A.tshape(1)], lambda ix: A.fromintegral(A.i32, A.f32, A.index(a, A.vexp(ix)))),
        A.lam([A.Int], lambda i: A.fromintegral(A.i32, A.f32, A.linearindex(a, i))))))
    assert np.array_equal(gpu_ctx.compile(conv)(xi), np.cumsum(xi).astype(np.float32))   # (sums below 2^24: exact)


@pytest.mark.parametrize("rows,n", [(3, 16384 * 17), (5, 16384 * 16 + 8), (2, 16384 * 20 + 4)])
def test_several_rows(gpu_ctx, knobs, rows, n):
    # every row starts at a multiple of 16 bytes; rows end in partial tiles, which a second launch takes
    knobs("scan_tiles", 4)
    x = np.random.default_rng(rows).integers(-1000, 1000, (rows, n)).astype(np.int64)
    dx = gpu_ctx.to_device(x, A.tarray(2, A.i64))
    assert np.array_equal(gpu_ctx.compile(P.scanl1_sum(A.i64, 2)).execute(dx).to_host(), np.cumsum(x, axis=1))
    got = gpu_ctx.compile(P.scan_sum("l", A.i64, 2, 7)).execute(dx).to_host()
    assert np.array_equal(got, np.concatenate([np.full((rows, 1), 7), 7 + np.cumsum(x, axis=1)], axis=1))
    body, total = [p.to_host() for p in gpu_ctx.compile(P.scan_prime_sum("l", A.i64, 2, 1)).execute(dx).parts()]
    inc = 1 + np.cumsum(x, axis=1)
    assert np.array_equal(body, np.concatenate([np.full((rows, 1), 1), inc[:, :-1]], axis=1)) and np.array_equal(total, inc[:, -1])


def test_rows_that_are_not_16_byte_multiples_keep_the_other_kernels(gpu_ctx, knobs):
    knobs("scan_tiles", 4)
    x = np.random.default_rng(1).integers(-1000, 1000, (3, 28672 * 16 + 3)).astype(np.int32)
    assert np.array_equal(gpu_ctx.compile(P.scanl1_sum(A.i32, 2))(x), np.cumsum(x, axis=1, dtype=np.int32))


def test_an_operator_that_is_not_commutative(gpu_ctx, knobs):
    # a (+) b = b if b /= 0 else a ("the last non-zero value so far"): associative, not
    # commutative, so any tile, wave or chunk combined in the wrong order shows
    f = A.lam([A.Int, A.Int], lambda a, b: A.cond(A.neq(A.Int, b, A.constI(0)), b, a))
    prog = A.alam([A.tarray(1, A.Int)], lambda xs: A.scan("l", f, None, xs))
    rng = np.random.default_rng(5)
    n = 16384 * 70 + 999
    x = rng.integers(1, 1 << 40, n).astype(np.int64)
    x[rng.random(n) < 0.9995] = 0            # long stretches of zeros: values travel across many tiles
    x[0] = 17
    idx = np.maximum.accumulate(np.where(x != 0, np.arange(n), 0))
    want = x[idx]
    run = gpu_ctx.compile(prog)
    for tiles in (1, 4):
        knobs("scan_tiles", tiles)
        assert np.array_equal(run(x), want), tiles


def test_a_function_that_reads_a_second_array(gpu_ctx, knobs):
    # the combination indexes a table (tests/progs.py table_scan): the kernel's environment holds
    # an array besides the operand, and every value the function sees must be a value of the array
    knobs("scan_tiles", 4)
    k = 7
    tbl = np.array([(a + b) % k for a in range(k) for b in range(k)], np.int64)
    rng = np.random.default_rng(123)
    for kind in ("scan1", "scan"):
        run = gpu_ctx.compile(Q.table_scan(k, "l", kind))
        for n in (16384 * 16, 16384 * 33 + 5):
            x = rng.integers(0, k, n).astype(np.int64)
            inc = np.cumsum(x) % k
            want = inc if kind == "scan1" else np.concatenate([[0], inc])
            assert np.array_equal(run(tbl, x), want), (kind, n)


def test_full_size_against_the_other_variant(gpu_ctx, knobs):
    # the headline workloads through both kernels: Int64 bit for bit, Float32 inside the configuration's bound
    n = 1 << 28
    x = W.uniform_int(n, 20240601)
    run = gpu_ctx.compile(P.scanl1_sum(A.i64))
    dx = gpu_ctx.to_device(x, A.tarray(1, A.i64))
    knobs("scan_tiles", 4)
    a = run.execute(dx).to_host()
    assert np.array_equal(a, np.cumsum(x))
    del a, dx, x
    y = W.uniform_f32(n, 11, 0.0, 1.0)
    runf = gpu_ctx.compile(P.scanl1_sum(A.f32))
    dy = gpu_ctx.to_device(y, A.tarray(1, A.f32))
    got = runf.execute(dy).to_host()
    ref = np.cumsum(y, dtype=np.float64)
    assert np.all(np.abs(got - ref) <= 1e-4 * ref)     # the inputs are non-negative: sum |x_i| is the prefix itself


def test_lookback_wait_is_bounded_in_the_pipelined_kernel(gpu_ctx, knobs):
    # as for the other kernels: a ticket base that lags by 3 numbers every tile 3 too high, the first
    # tiles wait for predecessors that never run and give up after 50 polls; every workgroup ends,
    # the error is raised by the next wait on the stream and the context works afterwards
    knobs("scan_tiles", 4)
    x = W.uniform_int(16384 * 40, 3)
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

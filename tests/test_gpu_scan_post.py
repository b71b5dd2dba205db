"""map g (scan f z xs) with the scan written out as the map's operand: the scan applies g as it
stores its results (no second launch, no array between the two), where g reads no arrays.
The results must be those of the two launches, for every kernel a scan may take."""
from __future__ import annotations

import numpy as np
import pytest

from accelerate_amd import ir as A
from accelerate_amd import programs as P

pytestmark = pytest.mark.gpu

I64, F32 = A.i64, A.f32


def _launches(ctx, run, *args):
    ctx.sync()
    before = ctx.stat("launches")
    out = run(*args)
    return out, ctx.stat("launches") - before


def _halved(direction="l", seed=None, rank=1):
    # the element type changes on the way out: Int64 sums leave as Float32 halves
    g = A.lam([I64], lambda v: A.mul(F32, A.fromintegral(I64, F32, v), A.const(F32, 0.5)))
    z = None if seed is None else A.const(I64, seed)
    return A.alam([A.tarray(rank, I64)], lambda xs: A.map_(F32, g, A.scan(direction, P._binop(A.add, I64), z, xs)))


SHAPES = [(1,), (300,), (5000,), (1 << 20,), ((1 << 22) + 3,), (3000, 17), (40, 3000), (3, 70001)]


@pytest.mark.parametrize("shape", SHAPES, ids=lambda s: "x".join(map(str, s)))
@pytest.mark.parametrize("post", [1, 0], ids=["applied-by-the-scan", "own-launch"])
def test_a_function_applied_to_the_results(gpu_ctx, knobs, shape, post):
    knobs("scan_post", post)
    rank = len(shape)
    x = np.random.default_rng(len(shape) * 7 + shape[-1] % 13).integers(-1000, 1000, shape).astype(np.int64)
    run = gpu_ctx.compile(_halved(rank=rank))
    got, launches = _launches(gpu_ctx, run, x)
    assert np.array_equal(got, np.cumsum(x, axis=-1).astype(np.float32) * np.float32(0.5))
    assert launches == (1 if post else 2)
    # a right scan with a seed: one more element per row, the seed goes through the function too
    run = gpu_ctx.compile(_halved("r", 9, rank))
    want = np.concatenate([9 + np.cumsum(x[..., ::-1], axis=-1)[..., ::-1], np.full(shape[:-1] + (1,), 9)], axis=-1)
    assert np.array_equal(run(x), want.astype(np.float32) * np.float32(0.5))


@pytest.mark.parametrize("tiles", [0, 1, 2, 3])
def test_under_every_tile_size(gpu_ctx, knobs, tiles):
    knobs("scan_tiles", tiles)
    x = np.random.default_rng(tiles).integers(-1000, 1000, (37, 900)).astype(np.int64)
    assert np.array_equal(gpu_ctx.compile(_halved(rank=2))(x), np.cumsum(x, axis=1).astype(np.float32) * np.float32(0.5))


def test_one_value_in_two_out_and_two_in_one_out(gpu_ctx):
    # scalar sums leave as pairs (v, -v) ...
    T2 = A.ttup(I64, I64)
    g = A.lam([I64], lambda v: A.tup(v, A.sub(I64, A.const(I64, 0), v)))
    prog = A.alam([A.tarray(1, I64)], lambda xs: A.map_(T2, g, A.scan("l", P._binop(A.add, I64), A.const(I64, 4), xs)))
    x = np.random.default_rng(2).integers(-1000, 1000, 200_003).astype(np.int64)
    a, b = gpu_ctx.compile(prog)(x)
    want = np.concatenate([[4], 4 + np.cumsum(x)])
    assert np.array_equal(a, want) and np.array_equal(b, -want)
    # ... and pairs (sum, maximum) leave as their difference
    sh1 = A.tshape(1)

    def both(xs):
        src = A.delayed(A.tarray(1, T2), A.shape(xs), A.lam([sh1], lambda ix: A.tup(A.index(xs, A.vexp(ix)), A.index(xs, A.vexp(ix)))),
                        A.lam([A.Int], lambda i: A.tup(A.linearindex(xs, i), A.linearindex(xs, i))))

        def f(p, q):
            (ps, pm), (qs, qm) = A.untup(p), A.untup(q)
            return A.tup(A.add(I64, ps, qs), A.max_(I64, pm, qm))
        h = A.lam([T2], lambda v: A.sub(I64, A.untup(v)[0], A.untup(v)[1]))
        return A.map_(I64, h, A.scan("l", A.lam([T2, T2], f), None, src))

    got = gpu_ctx.compile(A.alam([A.tarray(1, I64)], both))(x)
    assert np.array_equal(got, np.cumsum(x) - np.maximum.accumulate(x))


def test_a_function_that_reads_an_array_keeps_its_own_launch(gpu_ctx):
    g = lambda ys: A.lam([I64], lambda v: A.add(I64, v, A.index(ys, A.sh(A.constI(1)))))
    prog = A.alam([A.tarray(1, I64), A.tarray(1, I64)],
                  lambda xs, ys: A.map_(I64, g(ys), A.scan("l", P._binop(A.add, I64), None, xs)))
    x = np.arange(100_000, dtype=np.int64)
    y = np.array([5, 70, 900], dtype=np.int64)
    got, launches = _launches(gpu_ctx, gpu_ctx.compile(prog), x, y)
    assert np.array_equal(got, np.cumsum(x) + 70) and launches == 2


def test_an_operand_inside_an_operand_is_evaluated_once(gpu_ctx):
    # scan over (map over (map xs)), both maps written out as operands: every variant of the scan
    # plans its operand, whose own operand must still be listed -- and run -- once
    inc = A.lam([I64], lambda v: A.add(I64, v, A.const(I64, 1)))
    prog = A.alam([A.tarray(1, I64)],
                  lambda xs: A.scan("l", P._binop(A.add, I64), None, A.map_(I64, inc, A.map_(I64, inc, xs))))
    x = np.arange(50_000, dtype=np.int64)
    got, launches = _launches(gpu_ctx, gpu_ctx.compile(prog), x)
    assert np.array_equal(got, np.cumsum(x + 2)) and launches == 3

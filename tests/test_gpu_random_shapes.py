"""Folds, scans, segmented folds, transpositions and histograms over shapes drawn at random around
the sizes where the kernels change their ways (powers of two and tile sizes, give or take a few
elements; one row, a few rows, very many short ones), under launch-time choices drawn at random
too, against numpy.  Integer data, so every result is exact.  ACCHIP_RANDOM_SHAPES sets the
number of draws (default 300), ACCHIP_RANDOM_MOST the size of the largest array, ACCHIP_RANDOM_SEED
another sequence."""
from __future__ import annotations

import os

import numpy as np
import pytest

from accelerate_amd import ir as A
from accelerate_amd import programs as P

from . import progs as Q

pytestmark = pytest.mark.gpu

I64, I32 = A.i64, A.i32
DRAWS = int(os.environ.get("ACCHIP_RANDOM_SHAPES", "300"))
MOST = int(os.environ.get("ACCHIP_RANDOM_MOST", str(1 << 22)))   # elements of the largest array drawn
SEED = int(os.environ.get("ACCHIP_RANDOM_SEED", "0"))             # added to every test's seed


def _length(rng, most):
    base = int(2 ** (np.log2(most) * rng.uniform(0, 1) ** 0.5))   # more long than short
    if rng.random() < 0.6:
        base = 1 << int(round(np.log2(max(base, 1))))          # a power of two ...
        if rng.random() < 0.3:
            base = base // 4 * 7 // 2 or 1                     # ... or 7/8 of one (tiles of 112 bytes per lane)
    return max(1, min(most, base + int(rng.integers(-3, 4))))


def _shape(rng, most=MOST):
    kind = rng.integers(0, 4)
    if kind == 0:
        return (_length(rng, most),)
    n = _length(rng, most if kind == 1 else 1 << 12)
    rows = _length(rng, max(1, most // n))
    if kind == 3 and rows * n * 4 <= most:
        return (int(rng.integers(1, 5)), rows, n)
    return (rows, n)


_last = A.lam([I64, I64], lambda p, q: A.cond(A.neq(I64, q, A.constI(0)), q, p))
KNOBS = {"scan_tiles": [0, 0, 0, 1, 2, 3, 4], "fold_rows": [-1, -1, -1, 0, 1, 2], "scan_ticketless": [1, 1, 0],
         "fold_staged": [1, 1, 0], "fold_one_launch": [1, 1, 0], "fold_target": [2048, 2048, 64, 7]}


def _last_nonzero(x):
    n = x.shape[-1]
    idx = np.where(x != 0, np.arange(n), -1).max(axis=-1)
    return np.where(idx >= 0, np.take_along_axis(x, np.maximum(idx, 0)[..., None], axis=-1)[..., 0], 0)


def _running_last_nonzero(x):
    n = x.shape[-1]
    idx = np.maximum.accumulate(np.where(x != 0, np.arange(n), -1), axis=-1)
    return np.where(idx >= 0, np.take_along_axis(x, np.maximum(idx, 0), axis=-1), 0)


def test_shapes_and_launch_choices_drawn_at_random(gpu_ctx, knobs):
    rng = np.random.default_rng(20240613 + SEED)
    progs = {}

    def prog(key, make):
        if key not in progs:
            progs[key] = gpu_ctx.compile(make())
        return progs[key]

    for draw in range(DRAWS):
        setting = {k: int(rng.choice(v)) for k, v in KNOBS.items()}
        for k, v in setting.items():
            knobs(k, v)
        shape = _shape(rng)
        rank = len(shape)
        if setting["scan_tiles"] in (1, 4) and int(np.prod(shape[:-1])) > (1 << 21):
            knobs("scan_tiles", 0)   # a 1024-thread workgroup per row: more threads than one launch holds (refused)
        what = ["fold", "fold_last", "scanl1", "scanl", "scanr_prime", "scan_last", "transpose", "histogram", "foldseg"][rng.integers(0, 9)]
        where = (draw, what, shape, setting)
        x = rng.integers(-1000, 1000, shape).astype(np.int64)
        if what == "fold":
            got = prog(("fold", rank), lambda: P.fold_sum(I64, rank, 5))(x)
            assert np.array_equal(got, 5 + x.sum(axis=-1)), where
        elif what == "fold_last":
            x[rng.random(shape) < 0.8] = 0
            got = prog(("fold_last", rank), lambda: A.alam([A.tarray(rank, I64)], lambda xs: A.fold(_last, A.constI(0), xs)))(x)
            assert np.array_equal(got, _last_nonzero(x)), where
        elif what == "scanl1":
            got = prog(("scanl1", rank), lambda: P.scanl1_sum(I64, rank))(x)
            assert np.array_equal(got, np.cumsum(x, axis=-1)), where
        elif what == "scanl":
            x32 = x.astype(np.int32)
            got = prog(("scanl", rank), lambda: P.scan_sum("l", I32, rank, 3))(x32)
            want = np.concatenate([np.full(shape[:-1] + (1,), 3), 3 + np.cumsum(x, axis=-1)], axis=-1).astype(np.int32)
            assert np.array_equal(got, want), where
        elif what == "scanr_prime":
            body, total = prog(("scanr'", rank), lambda: P.scan_prime_sum("r", I64, rank, 1))(x)
            inc = 1 + np.cumsum(x[..., ::-1], axis=-1)[..., ::-1]
            want = np.concatenate([inc[..., 1:], np.full(shape[:-1] + (1,), 1)], axis=-1)
            assert np.array_equal(body, want) and np.array_equal(total, inc[..., 0]), where
        elif what == "scan_last":
            x[rng.random(shape) < 0.9] = 0
            got = prog(("scan_last", rank), lambda: A.alam([A.tarray(rank, I64)], lambda xs: A.scan("l", _last, None, xs)))(x)
            assert np.array_equal(got, _running_last_nonzero(x)), where
        elif what == "transpose":
            if rank != 2:
                continue
            got = prog(("transpose",), lambda: Q.transpose(I64))(x)
            assert np.array_equal(got, x.T), where
        elif what == "histogram":
            # sums into nbins elements (sizes that are set when the program runs); a negative target drops its source
            nbins = _length(rng, 1 << 18)
            to = rng.integers(-1, nbins, shape)
            dfl = rng.integers(-5, 5, nbins).astype(np.int64)
            got = prog(("accumulate", rank), lambda: Q.accumulate(I64, rank, 1))(x, to.reshape(-1), dfl)
            want = dfl.copy()
            np.add.at(want, to[to >= 0], x[to >= 0])
            assert np.array_equal(got, want), where + (nbins,)
        else:
            n = shape[-1]
            cuts = np.sort(rng.integers(0, n + 1, int(rng.integers(0, max(1, min(n, 5000))))))
            lens = np.diff(np.concatenate([[0], cuts, [n]])).astype(np.int32)        # empty segments included
            x32 = x.astype(np.int32)
            got = prog(("foldseg", rank), lambda: P.foldseg_sum(I32, I32, rank, 2))(x32, lens)
            ends = np.cumsum(lens)
            cs = np.concatenate([np.zeros(shape[:-1] + (1,), np.int64), np.cumsum(x, axis=-1)], axis=-1)
            want = (2 + cs[..., ends] - cs[..., ends - lens]).astype(np.int32)
            assert np.array_equal(got, want), where


def _weighted_reference(x, widths, mode, fill):
    """numpy restatement of progs.stencil_weighted: tap number k (1-based, the outermost component
    of the stencil walking the slowest index) weighs k"""
    rank = x.ndim
    halo = [w // 2 for w in widths]
    pad = [(h, h) for h in halo]
    if mode == "constant":
        xp = np.pad(x, pad, mode="constant", constant_values=fill)
    else:
        xp = np.pad(x, pad, mode={"clamp": "edge", "mirror": "reflect", "wrap": "wrap"}[mode])
    out = np.zeros_like(x)
    k = 0
    for offs in np.ndindex(*widths):
        k += 1
        sl = tuple(slice(o, o + n) for o, n in zip(offs, x.shape))
        out += k * xp[sl]
    return out


def test_stencil_shapes_drawn_at_random(gpu_ctx, knobs):
    # rank 2 (tiles in LDS) and rank 3 (a ring of planes in LDS) with every boundary condition, on
    # extents from a single row or plane up to several tiles, mirrored and wrapped halos included
    # (np.pad needs an extent of at least 2 to mirror)
    rng = np.random.default_rng(20240614 + SEED)
    progs = {}
    for draw in range(max(20, DRAWS // 5)):
        rank = int(rng.integers(2, 4))
        mode = ["clamp", "mirror", "wrap", "constant"][rng.integers(0, 4)]
        widths = [3] * rank if rng.random() < 0.7 else ([5, 3] if rank == 2 else [3, 5, 3])
        most = 1 << (21 if rank == 2 else 20)
        shape = []
        left = most
        for d in range(rank):
            n = max(widths[d] // 2 + 1, _length(rng, max(2, min(left, 3000 if d else 600))))
            shape.append(n)
            left = max(2, left // n)
        shape = tuple(shape)
        knobs("stencil_chain", int(rng.choice([0, 0, 1, 3])))
        key = (rank, mode, tuple(widths))
        if key not in progs:
            b = A.constant(I64, 7) if mode == "constant" else mode
            progs[key] = gpu_ctx.compile(Q.stencil_weighted(I64, widths, b))
        x = rng.integers(-100, 100, shape).astype(np.int64)
        got = progs[key](x)
        assert np.array_equal(got, _weighted_reference(x, widths, mode, 7)), (draw, shape, mode, widths)


def _merge_two_smallest():
    """permute with Issue137's merge into given defaults: an element ends as the two smallest of
    the values sent to it and its own two (needs the lock: no component stands alone)"""
    t2 = A.ttup(I64, I64)
    sh1 = A.tshape(1)
    big = A.const(I64, 1 << 40)

    def comb(p, q):
        a1, a2 = A.untup(p)
        b1, b2 = A.untup(q)
        return A.cond(A.lte(I64, a1, b1), A.tup(a1, A.min_(I64, a2, b1)), A.tup(b1, A.min_(I64, b2, a1)))

    def body(xs, to, dfl):
        src = A.delayed(A.tarray(1, t2), A.shape(xs), A.lam([sh1], lambda ix: A.tup(A.index(xs, A.vexp(ix)), big)),
                        A.lam([A.Int], lambda i: A.tup(A.linearindex(xs, i), big)))
        tgt = lambda ix: A.cond(A.lt(A.Int, A.index(to, A.vexp(ix)), A.constI(0)), A.nothing(sh1),
                                A.just(A.sh(A.index(to, A.vexp(ix)))))
        return A.permute(A.lam([t2, t2], comb), dfl, A.lam([sh1], tgt), src)

    return A.alam([A.tarray(1, I64), A.tarray(1, A.Int), A.tarray(1, t2)], body)


def test_permutes_of_every_kind_over_sizes_drawn_at_random(gpu_ctx, knobs):
    # one hardware atomic (sum), a compare-and-swap loop (product), one atomic per component (sum
    # and maximum of pairs), the lock (two smallest): sources from a handful to millions, destinations
    # from one element to more than the private copies take, some sources dropped, some elements popular
    rng = np.random.default_rng(20240615 + SEED)
    sh1 = A.tshape(1)
    t2 = A.ttup(I64, I64)
    drop = lambda to: lambda ix: A.cond(A.lt(A.Int, A.index(to, A.vexp(ix)), A.constI(0)), A.nothing(sh1),
                                       A.just(A.sh(A.index(to, A.vexp(ix)))))
    scalar = lambda op: A.alam([A.tarray(1, I64), A.tarray(1, A.Int), A.tarray(1, I64)], lambda xs, to, dfl: A.permute(
        Q.binop(op, I64), dfl, A.lam([sh1], drop(to)), xs))
    sum_max = A.alam([A.tarray(1, t2), A.tarray(1, A.Int), A.tarray(1, t2)], lambda xs, to, dfl: A.permute(
        A.lam([t2, t2], lambda p, q: A.tup(A.add(I64, A.untup(p)[0], A.untup(q)[0]), A.max_(I64, A.untup(p)[1], A.untup(q)[1]))),
        dfl, A.lam([sh1], drop(to)), xs))
    progs = {"sum": gpu_ctx.compile(scalar(A.add)), "product": gpu_ctx.compile(scalar(A.mul)),
             "sum_max": gpu_ctx.compile(sum_max), "two_smallest": gpu_ctx.compile(_merge_two_smallest())}
    for draw in range(max(20, DRAWS // 3)):
        what = list(progs)[rng.integers(0, 4)]
        n = _length(rng, 1 << 21)
        nbins = _length(rng, 1 << 19)
        parts = int(rng.choice([128, 128, 128, 2, 0]))
        if what in ("two_smallest", "product") and n > 3000 * nbins:
            parts = 128   # (without the private copies these sources would take turns in memory: thousands per element, 20 µs a turn)
        knobs("permute_parts", parts)
        to = rng.integers(-1, nbins, n)
        if rng.random() < 0.5:
            # a popular element: a fifth of the sources -- a couple of thousand where they take turns at
            # a lock or a compare-and-swap loop in memory (no private copies: few sources, a large
            # destination, or the copies switched off)
            share = 0.2
            if what in ("two_smallest", "product") and (parts != 128 or nbins > 100_000 or n < (1 << 20)):
                share = min(share, 2000 / n)
            to[rng.random(n) < share] = int(rng.integers(0, nbins))
        keep = to >= 0
        where = (draw, what, n, nbins)
        if what == "sum":
            x = rng.integers(-1000, 1000, n).astype(np.int64)
            dfl = rng.integers(-5, 5, nbins).astype(np.int64)
            want = dfl.copy()
            np.add.at(want, to[keep], x[keep])
            assert np.array_equal(progs[what](x, to, dfl), want), where
        elif what == "product":
            x = rng.integers(0, 1 << 62, n, dtype=np.int64) | 1
            dfl = rng.integers(1, 1000, nbins).astype(np.int64)
            want = dfl.astype(np.uint64)
            np.multiply.at(want, to[keep], x[keep].astype(np.uint64))
            assert np.array_equal(progs[what](x, to, dfl).astype(np.uint64), want), where
        elif what == "sum_max":
            x = rng.integers(-1000, 1000, n).astype(np.int64)
            y = rng.integers(-1000, 1000, n).astype(np.int64)
            d0 = rng.integers(-5, 5, nbins).astype(np.int64)
            d1 = rng.integers(-1000, 1000, nbins).astype(np.int64)
            w0, w1 = d0.copy(), d1.copy()
            np.add.at(w0, to[keep], x[keep])
            np.maximum.at(w1, to[keep], y[keep])
            a, b = progs[what](gpu_ctx.to_device((x, y), A.tarray(1, t2)), to, gpu_ctx.to_device((d0, d1), A.tarray(1, t2)))
            assert np.array_equal(a, w0) and np.array_equal(b, w1), where
        else:
            x = rng.integers(0, 1 << 30, n, dtype=np.int64)
            d0 = rng.integers(0, 1 << 31, nbins, dtype=np.int64)
            d1 = d0 + rng.integers(0, 1 << 31, nbins, dtype=np.int64)        # a pair is (smallest, second smallest)
            vals = np.concatenate([x[keep], d0, d1])
            bins = np.concatenate([to[keep], np.arange(nbins), np.arange(nbins)])
            order = np.lexsort((vals, bins))
            vs, bs = vals[order], bins[order]
            first = np.searchsorted(bs, np.arange(nbins))
            a, b = progs[what](x, to, gpu_ctx.to_device((d0, d1), A.tarray(1, t2)))
            assert np.array_equal(a, vs[first]) and np.array_equal(b, vs[first + 1]), where


def test_scans_with_producers_and_epilogues_over_shapes_drawn_at_random(gpu_ctx, knobs):
    # a producer fused into the scan (of one array: it may ride in the pipelined kernel; of two: it
    # may not), a function applied to the results as they are stored, pairs as elements, right scans
    rng = np.random.default_rng(20240616 + SEED)
    t2 = A.ttup(I64, I64)
    progs = {}

    def fused(rank, two):
        shr = A.tshape(rank)
        g = (lambda v, u: A.add(I64, v, u)) if two else (lambda v: A.add(I64, A.mul(I64, v, A.const(I64, 2)), A.const(I64, 1)))

        def body(a, *more):
            at = lambda ix: g(A.index(a, A.vexp(ix)), *[A.index(m, A.vexp(ix)) for m in more])
            lin = lambda i: g(A.linearindex(a, i), *[A.linearindex(m, i) for m in more])
            return A.scan("l", P._binop(A.add, I64), None, A.delayed(A.tarray(rank, I64), A.shape(a), A.lam([shr], at), A.lam([A.Int], lin)))
        return A.alam([A.tarray(rank, I64)] * (2 if two else 1), body)

    def pairs(rank, direction):
        f = A.lam([t2, t2], lambda p, q: A.tup(A.add(I64, A.untup(p)[0], A.untup(q)[0]), A.max_(I64, A.untup(p)[1], A.untup(q)[1])))
        return A.alam([A.tarray(rank, t2)], lambda xs: A.scan(direction, f, None, xs))

    def halved(rank):
        g = A.lam([I64], lambda v: A.sub(I32, A.fromintegral(I64, I32, v), A.const(I32, 1)))
        return A.alam([A.tarray(rank, I64)], lambda xs: A.map_(I32, g, A.scan("r", P._binop(A.add, I64), A.const(I64, 2), xs)))

    def prog(key, make):
        if key not in progs:
            progs[key] = gpu_ctx.compile(make())
        return progs[key]

    for draw in range(max(20, DRAWS // 3)):
        tiles = int(rng.choice([0, 0, 0, 1, 2, 3, 4]))
        shape = _shape(rng)
        if len(shape) == 3:
            shape = shape[1:]
        rank = len(shape)
        if tiles in (1, 4) and int(np.prod(shape[:-1])) > (1 << 21):
            tiles = 0
        knobs("scan_tiles", tiles)
        knobs("scan_post", int(rng.choice([1, 1, 0])))
        what = ["fused1", "fused2", "pairs_l", "pairs_r", "halved"][rng.integers(0, 5)]
        where = (draw, what, shape, tiles)
        x = rng.integers(-1000, 1000, shape).astype(np.int64)
        y = rng.integers(-1000, 1000, shape).astype(np.int64)
        if what == "fused1":
            assert np.array_equal(prog((what, rank), lambda: fused(rank, False))(x), np.cumsum(2 * x + 1, axis=-1)), where
        elif what == "fused2":
            assert np.array_equal(prog((what, rank), lambda: fused(rank, True))(x, y), np.cumsum(x + y, axis=-1)), where
        elif what in ("pairs_l", "pairs_r"):
            d = what[-1]
            a, b = prog((what, rank), lambda: pairs(rank, d))(gpu_ctx.to_device((x, y), A.tarray(rank, t2)))
            if d == "l":
                wa, wb = np.cumsum(x, axis=-1), np.maximum.accumulate(y, axis=-1)
            else:
                wa = np.cumsum(x[..., ::-1], axis=-1)[..., ::-1]
                wb = np.maximum.accumulate(y[..., ::-1], axis=-1)[..., ::-1]
            assert np.array_equal(a, wa) and np.array_equal(b, wb), where
        else:
            inc = 2 + np.cumsum(x[..., ::-1], axis=-1)[..., ::-1]
            want = np.concatenate([inc, np.full(shape[:-1] + (1,), 2)], axis=-1).astype(np.int32) - np.int32(1)
            assert np.array_equal(prog((what, rank), lambda: halved(rank))(x), want), where


def test_axis_permutations_over_extents_drawn_at_random(gpu_ctx, knobs):
    # transpositions of matrices and the six orders of the dimensions of rank 3, extents from 1 to
    # a few thousand: tiles of the plane of the two dimensions involved, ragged on every side
    rng = np.random.default_rng(20240617 + SEED)
    perms = [(0, 2, 1), (1, 0, 2), (2, 1, 0), (1, 2, 0), (2, 0, 1)]
    progs = {}
    for draw in range(max(20, DRAWS // 3)):
        knobs("map_tiled", int(rng.choice([-1, -1, -1, 0, 1])))
        if rng.random() < 0.4:
            shape = (_length(rng, 5000), _length(rng, 5000))
            while shape[0] * shape[1] > (1 << 22):
                shape = (shape[0] // 2 + 1, shape[1])
            x = rng.integers(-1000, 1000, shape).astype(np.int64)
            if "t" not in progs:
                progs["t"] = gpu_ctx.compile(Q.transpose(I64))
            assert np.array_equal(progs["t"](x), x.T), (draw, shape)
            continue
        pm = perms[rng.integers(0, len(perms))]
        shape = tuple(_length(rng, 300) for _ in range(3))
        x = rng.integers(-1000, 1000, shape).astype(np.int32)
        if pm not in progs:
            inv = [pm.index(k) for k in range(3)]
            progs[pm] = gpu_ctx.compile(Q.reindex(3, lambda dd, pm=pm: [dd()[pm[0]], dd()[pm[1]], dd()[pm[2]]],
                                                  lambda ix, dd, inv=inv: [ix[inv[0]], ix[inv[1]], ix[inv[2]]], I32))
        assert np.array_equal(progs[pm](x), x.transpose(pm)), (draw, shape, pm)

"""The LDS-privatised permute path (many sources, small destination, hardware-atomic
combination) against numpy's unbuffered ufunc.at, which applies the updates one by one in
source order exactly like permuteOp (Interpreter.hs:585-624).  Integer results bit-exact;
the Float32 case sums multiples of 1/4, which are exact in any order."""
import numpy as np
import pytest

from accelerate_amd import hip
from accelerate_amd import ir as A

from . import progs as Q

N = (1 << 20) + 12345        # above the threshold that selects the privatised kernel


def lds_programs():
    """(id, program, numpy dtype, ufunc, destination size)"""
    out = []
    for ty, dt in ((A.i32, np.int32), (A.i64, np.int64), (A.f32, np.float32)):
        for dst in (100, 40000, 70000):     # 1 range, 2 ranges (4-byte), up to 5 ranges (8-byte)
            out.append(("add_%s_%d" % (ty, dst), Q.accumulate(ty, 1, 1), dt, np.add, dst))
    for name, op, uf in (("min", A.min_, np.minimum), ("max", A.max_, np.maximum), ("bxor", A.bxor, np.bitwise_xor)):
        out.append(("%s_i32_5000" % name, _combine_prog(op, A.i32), np.int32, uf, 5000))
    return out


def _combine_prog(op, ty):
    sh1 = A.tshape(1)
    return A.alam([A.tarray(1, ty), A.tarray(1, A.Int), A.tarray(1, ty)], lambda xs, to, dfl: A.permute(
        Q.binop(op, ty), dfl,
        A.lam([sh1], lambda ix: A.let(A.Int, A.index(to, A.vexp(ix)), lambda t: A.cond(
            A.lt(A.Int, t, A.constI(0)), A.nothing(sh1), A.just(A.sh(t))))), xs))


CASES = lds_programs()


@pytest.mark.gpu
@pytest.mark.parametrize("case", CASES, ids=[c[0] for c in CASES])
def test_privatised_permute_matches_sequential_updates(gpu_ctx, case):
    _, prog, dt, uf, dst = case
    rng = np.random.default_rng(dst)
    # skewed targets (hot destinations) and some dropped sources (negative target)
    to = np.minimum((rng.pareto(1.1, N) * 3).astype(np.int64), dst - 1)
    to[rng.random(N) < 0.05] = -1
    if dt == np.float32:
        xs = (rng.integers(-8, 9, N) / 4).astype(dt)
        dfl = (rng.integers(-8, 9, dst) / 4).astype(dt)
    else:
        xs = rng.integers(-1000, 1000, N).astype(dt)
        dfl = rng.integers(-1000, 1000, dst).astype(dt)
    got = gpu_ctx.compile(prog)(xs, to, dfl)
    ref = dfl.copy()
    keep = to >= 0
    uf.at(ref, to[keep], xs[keep])
    assert np.array_equal(got, ref)


@pytest.mark.gpu
@pytest.mark.parametrize("dst", [7, 300, 20000, 50000])
def test_privatised_permute_of_pairs(gpu_ctx, dst):
    # component-wise combinations of tuples keep one private array per component: sums of
    # (Int64, Int32 maximum) pairs and of Float32 pairs (quarters: exact in any order) into
    # 1 .. 5 ranges of the destination
    rng = np.random.default_rng(dst)
    to = np.minimum((rng.pareto(1.1, N) * 3).astype(np.int64), dst - 1)
    a, b = rng.integers(-1000, 1000, N).astype(np.int64), rng.integers(-1000, 1000, N).astype(np.int32)
    da, db = rng.integers(-1000, 1000, dst).astype(np.int64), rng.integers(-1000, 1000, dst).astype(np.int32)
    got = gpu_ctx.compile(Q.accumulate_pairs(A.i64, A.i32, A.max_))([a, b], to, [da, db])
    ra, rb = da.copy(), db.copy()
    np.add.at(ra, to, a)
    np.maximum.at(rb, to, b)
    assert np.array_equal(got[0], ra) and np.array_equal(got[1], rb)
    x, y = (rng.integers(-8, 9, N) / 4).astype(np.float32), (rng.integers(-8, 9, N) / 4).astype(np.float32)
    got = gpu_ctx.compile(Q.accumulate_pairs())([x, y], to, [np.zeros(dst, np.float32)] * 2)
    rx, ry = np.zeros(dst, np.float64), np.zeros(dst, np.float64)
    np.add.at(rx, to, x)
    np.add.at(ry, to, y)
    assert np.array_equal(got[0], rx.astype(np.float32)) and np.array_equal(got[1], ry.astype(np.float32))


def _histogram_with_drops(nbins, ty=A.i32, value=1):
    """permute (+) zeros (\\ix -> if k < 0 then Nothing else Just k) (fill value): a constant per source"""
    sh1 = A.tshape(1)
    return A.alam([A.tarray(1, A.Int)], lambda keys: A.permute(
        Q.binop(A.add, ty),
        A.generate(A.tarray(1, ty), A.sh(nbins), A.lam([sh1], lambda ix: A.const(ty, 0))),
        A.lam([sh1], lambda ix: A.let(A.Int, A.index(keys, A.vexp(ix)), lambda t: A.cond(
            A.lt(A.Int, t, A.constI(0)), A.nothing(sh1), A.just(A.sh(t))))),
        A.delayed(A.tarray(1, ty), A.shape(keys), A.lam([sh1], lambda ix: A.const(ty, value)),
                  A.lam([A.Int], lambda i: A.const(ty, value)))))


COUNT_KEYS = ["one_key", "two_keys_one_word", "last_bin", "sorted", "zipf", "uniform", "drops"]


@pytest.mark.gpu
@pytest.mark.parametrize("keys_kind", COUNT_KEYS)
@pytest.mark.parametrize("nbins,ty,value", [(1 << 16, A.i32, 1), (40000, A.i64, -3), (65537, A.i32, 7), (300000, A.u32, 1),
                                            (1 << 16, A.i32, 0x7fffffff)])
def test_counting_permute_matches_bincount(gpu_ctx, keys_kind, nbins, ty, value):
    # a sum of one constant per source is counted in 16-bit LDS counters that are relieved of 32768
    # whenever they reach it: inputs that drive single counters through many such crossings (one key;
    # two keys whose counters share a word), the range's last element, and ordinary distributions,
    # over one and several ranges of the destination; sums wrap like the reference's fixed-width types
    n = (1 << 22) + 4321
    rng = np.random.default_rng(nbins)
    if keys_kind == "one_key":
        keys = np.full(n, min(12345, nbins - 1), np.int64)
    elif keys_kind == "two_keys_one_word":
        keys = np.where(rng.random(n) < 0.5, 77, 77 + 32768).astype(np.int64) % nbins
    elif keys_kind == "last_bin":
        keys = np.where(rng.random(n) < 0.7, nbins - 1, 65535 % nbins).astype(np.int64)
    elif keys_kind == "sorted":
        keys = np.sort(rng.integers(0, nbins, n)).astype(np.int64)
    elif keys_kind == "zipf":
        keys = np.minimum(rng.zipf(1.1, n) - 1, nbins - 1).astype(np.int64)
    elif keys_kind == "uniform":
        keys = rng.integers(0, nbins, n).astype(np.int64)
    else:
        keys = rng.integers(0, nbins, n).astype(np.int64)
        keys[rng.random(n) < 0.3] = -1
    got = gpu_ctx.compile(_histogram_with_drops(nbins, ty, value))(keys)
    dt = {"i32": np.int32, "i64": np.int64, "u32": np.uint32}[ty]
    counts = np.bincount(keys[keys >= 0], minlength=nbins).astype(np.int64)
    want = (counts * value).astype(np.int64).astype(dt)      # wraps to the element type
    assert got.dtype == dt and np.array_equal(got, want)


@pytest.mark.gpu
def test_counting_permute_agrees_with_the_atomic_paths(gpu_ctx, knobs):
    rng = np.random.default_rng(3)
    keys = np.minimum(rng.zipf(1.1, 1 << 22) - 1, 65535).astype(np.int64)
    prog = _histogram_with_drops(1 << 16)
    a = gpu_ctx.compile(prog)(keys)
    knobs("permute_count", 0)
    b = gpu_ctx.compile(prog)(keys)
    assert np.array_equal(a, b) and np.array_equal(a, np.bincount(keys, minlength=1 << 16))


def _histogram_of_narrow_keys(nbins, key_ty, drop_negative):
    """The same with keys of at most 32 bits widened by fromIntegral: the index test of the
    counting kernel then stays in 32 bits."""
    sh1 = A.tshape(1)

    def target(ix, keys):
        k = A.index(keys, A.vexp(ix))
        wide = A.fromintegral(key_ty, A.Int, k)
        if not drop_negative:
            return A.just(A.sh(wide))
        return A.let(A.Int, wide, lambda t: A.cond(A.lt(A.Int, t, A.constI(0)), A.nothing(sh1), A.just(A.sh(t))))

    return A.alam([A.tarray(1, key_ty)], lambda keys: A.permute(
        Q.binop(A.add, A.i32),
        A.generate(A.tarray(1, A.i32), A.sh(nbins), A.lam([sh1], lambda ix: A.const(A.i32, 0))),
        A.lam([sh1], lambda ix: target(ix, keys)),
        A.delayed(A.tarray(1, A.i32), A.shape(keys), A.lam([sh1], lambda ix: A.const(A.i32, 1)),
                  A.lam([A.Int], lambda i: A.const(A.i32, 1)))))


@pytest.mark.gpu
@pytest.mark.parametrize("key_ty,npt", [(A.i32, np.int32), (A.u32, np.uint32), (A.i16, np.int16), (A.u8, np.uint8)])
@pytest.mark.parametrize("nbins", [200, 1 << 16, 3 * 65536 + 5])
def test_counting_permute_with_narrow_keys(gpu_ctx, key_ty, npt, nbins):
    # targets inside one and several ranges, in the last element, and (signed keys, dropped by the
    # index function) below zero; pinned by numpy's bincount
    n = (1 << 21) + 77
    rng = np.random.default_rng(nbins + np.dtype(npt).itemsize)
    top = min(nbins, int(np.iinfo(npt).max) + 1)
    keys = rng.integers(0, top, n).astype(npt)
    keys[::1000] = top - 1
    signed = np.iinfo(npt).min < 0
    if signed:
        keys[rng.random(n) < 0.2] = -1
        keys[5] = np.iinfo(npt).min
    got = gpu_ctx.compile(_histogram_of_narrow_keys(nbins, key_ty, signed))(keys)
    k64 = keys.astype(np.int64)
    assert np.array_equal(got, np.bincount(k64[k64 >= 0], minlength=nbins).astype(np.int32))


@pytest.mark.gpu
@pytest.mark.parametrize("key_ty,npt,bad", [(A.i32, np.int32, -1), (A.i32, np.int32, 1 << 16), (A.u32, np.uint32, 0xffffffff),
                                            (A.i32, np.int32, -(1 << 31))])
def test_narrow_key_outside_the_destination_is_an_error(gpu_ctx, key_ty, npt, bad):
    # toIndex's bounds check (Shape.hs:98-106): reported by the next wait, nothing written for it
    keys = np.random.default_rng(4).integers(0, 1 << 16, 1 << 21).astype(npt)
    keys[12345] = npt(bad) if bad >= 0 else np.array(bad, np.int64).astype(npt)
    run = gpu_ctx.compile(_histogram_of_narrow_keys(1 << 16, key_ty, False))
    res = run.execute(gpu_ctx.to_device(keys, A.tarray(1, key_ty)))
    with pytest.raises(hip.AccError, match="index out of bounds"):
        gpu_ctx.sync()
    res.release()
    good = keys.copy()
    good[12345] = 7
    assert np.array_equal(run(good), np.bincount(good.astype(np.int64), minlength=1 << 16).astype(np.int32))


@pytest.mark.gpu
@pytest.mark.parametrize("fresh", [1, 0])
@pytest.mark.parametrize("keys_kind", ["one_key", "two_keys_one_word", "last_bin"])
@pytest.mark.parametrize("nbins", [1 << 16, 65537])
def test_counting_permute_relieves_counters_several_times(gpu_ctx, knobs, keys_kind, nbins, fresh):
    # 32 workgroups of 2^17 keys each: a counter that takes all of a workgroup's keys passes
    # 32768 four times.  With the defaults written by the summing kernel (fresh) the workgroup
    # notes each relief in its list; otherwise the relief goes to the destination at once.
    knobs("permute_groups", 32)
    knobs("permute_fresh", fresh)
    n = 1 << 22
    rng = np.random.default_rng(nbins + fresh)
    if keys_kind == "one_key":
        keys = np.full(n, 12345, np.int32)
    elif keys_kind == "two_keys_one_word":
        keys = np.where(rng.random(n) < 0.5, 77, 77 + 32768).astype(np.int32)
    else:
        keys = np.where(rng.random(n) < 0.7, nbins - 1, 65535).astype(np.int32)
    got = gpu_ctx.compile(_histogram_of_narrow_keys(nbins, A.i32, False))(keys)
    assert np.array_equal(got, np.bincount(keys, minlength=nbins).astype(np.int32))


@pytest.mark.gpu
def test_counting_permute_writes_constant_defaults_itself(gpu_ctx, knobs):
    # defaults of one constant other than zero, a constant other than one per source, a
    # destination that is not a whole number of ranges: every element must come out as
    # default + count * constant, also those no key points at
    sh1 = A.tshape(1)
    nbins, n = 70001, 1 << 21
    prog = A.alam([A.tarray(1, A.i32)], lambda keys: A.permute(
        Q.binop(A.add, A.i64),
        A.generate(A.tarray(1, A.i64), A.sh(nbins), A.lam([sh1], lambda ix: A.const(A.i64, -5))),
        A.lam([sh1], lambda ix: A.just(A.sh(A.fromintegral(A.i32, A.Int, A.index(keys, A.vexp(ix)))))),
        A.delayed(A.tarray(1, A.i64), A.shape(keys), A.lam([sh1], lambda ix: A.const(A.i64, 3)),
                  A.lam([A.Int], lambda i: A.const(A.i64, 3)))))
    keys = np.random.default_rng(9).integers(0, nbins - 1000, n).astype(np.int32)   # the last 1000 bins stay at the default
    want = np.bincount(keys, minlength=nbins).astype(np.int64) * 3 - 5
    for fresh in (1, 0):
        knobs("permute_fresh", fresh)
        assert np.array_equal(gpu_ctx.compile(prog)(keys), want)


# -- combinations that need the lock: private copies in LDS under LDS locks, combined by a second launch

def _two_smallest(nbins, a_ty=A.i64, b_ty=A.i64, big=1 << 40):
    """permute into (inf, inf) pairs: every element ends as the two smallest values sent to it (the
    merge of Issue137: associative and commutative, but no component is a function of its own
    component alone, so no hardware atomic fits); a negative target drops the source"""
    t2 = A.ttup(a_ty, b_ty)
    sh1 = A.tshape(1)
    inf_a, inf_b = A.const(a_ty, big), A.const(b_ty, big)
    conv = (lambda e: e) if a_ty == b_ty else (lambda e: A.fromintegral(a_ty, b_ty, e))
    back = (lambda e: e) if a_ty == b_ty else (lambda e: A.fromintegral(b_ty, a_ty, e))

    def comb(p, q):
        a1, a2 = A.untup(p)
        b1, b2 = A.untup(q)
        return A.cond(A.lte(a_ty, a1, b1), A.tup(a1, A.min_(b_ty, a2, conv(b1))), A.tup(b1, A.min_(b_ty, b2, conv(a1))))

    def body(xs, to):
        src = A.delayed(A.tarray(1, t2), A.shape(xs), A.lam([sh1], lambda ix: A.tup(A.index(xs, A.vexp(ix)), inf_b)),
                        A.lam([A.Int], lambda i: A.tup(A.linearindex(xs, i), inf_b)))
        tgt = lambda ix: A.cond(A.lt(A.Int, A.index(to, A.vexp(ix)), A.constI(0)), A.nothing(sh1),
                                A.just(A.sh(A.index(to, A.vexp(ix)))))
        return A.permute(A.lam([t2, t2], comb),
                         A.generate(A.tarray(1, t2), A.sh(nbins), A.lam([sh1], lambda ix: A.tup(inf_a, inf_b))),
                         A.lam([sh1], tgt), src)

    return A.alam([A.tarray(1, a_ty), A.tarray(1, A.Int)], body)


def _two_smallest_ref(x, to, nbins, big):
    keep = to >= 0
    x, to = x[keep], to[keep]
    order = np.lexsort((x, to))
    ts, xs = to[order], x[order]
    n = len(xs)
    first = np.searchsorted(ts, np.arange(nbins))
    cnt = np.diff(np.append(first, n))
    m1 = np.where(cnt > 0, xs[np.minimum(first, n - 1)], big)
    m2 = np.where(cnt > 1, xs[np.minimum(first + 1, n - 1)], big)
    return m1, m2


# 6553 elements of (Int64, Int64) and their state word fill 128 KiB of LDS: one range, two ranges,
# several, and more than the privatised kernel accepts (global locks)
@pytest.mark.gpu
@pytest.mark.parametrize("nbins", [1, 7, 384, 6553, 6554, 70000, 300000])
@pytest.mark.parametrize("order", ["fences", "waits"])
def test_locked_combination_through_private_copies(gpu_ctx, monkeypatch, nbins, order):
    if order == "fences":
        monkeypatch.setenv("ACCHIP_LOCK_ORDER", "fences")   # read when the kernel is generated
    rng = np.random.default_rng(nbins)
    n = N
    x = rng.integers(0, 1 << 30, n, dtype=np.int64)
    to = rng.integers(-1, nbins, n, dtype=np.int64)         # -1: dropped
    # a third of the sources want one element (a few thousand of them where the global locks serve: they take turns there)
    to[rng.random(n) < (0.3 if nbins <= 200000 else 0.002)] = nbins // 2
    a, b = gpu_ctx.compile(_two_smallest(nbins))(x, to)
    m1, m2 = _two_smallest_ref(x, to, nbins, 1 << 40)
    assert np.array_equal(a, m1) and np.array_equal(b, m2)


@pytest.mark.gpu
def test_locked_combination_few_sources_and_mixed_component_types(gpu_ctx):
    # below the threshold of the privatised kernel: global locks under contention
    rng = np.random.default_rng(8)
    x = rng.integers(0, 1 << 30, 3000, dtype=np.int64)
    to = rng.integers(0, 5, 3000, dtype=np.int64)
    a, b = gpu_ctx.compile(_two_smallest(5))(x, to)
    m1, m2 = _two_smallest_ref(x, to, 5, 1 << 40)
    assert np.array_equal(a, m1) and np.array_equal(b, m2)
    # (Int32, Int64) pairs: 16 bytes with the state word, 8192 elements per range
    n = N
    x = rng.integers(0, 1 << 30, n).astype(np.int32)
    for nbins in (8192, 8193):
        to = rng.integers(0, nbins, n, dtype=np.int64)
        a, b = gpu_ctx.compile(_two_smallest(nbins, A.i32, A.i64, 1 << 30))(x, to)
        m1, m2 = _two_smallest_ref(x.astype(np.int64), to, nbins, 1 << 30)
        assert np.array_equal(a, m1.astype(np.int32)) and np.array_equal(b, m2)


# -- scalar combinations without a hardware atomic (compare-and-swap loop): the same private copies

@pytest.mark.gpu
@pytest.mark.parametrize("nbins", [3, 10922, 10923, 60000, 200000])   # one range, two, six, and the CAS loop in memory
def test_products_through_private_copies(gpu_ctx, nbins):
    sh1 = A.tshape(1)
    prog = A.alam([A.tarray(1, A.i64), A.tarray(1, A.Int), A.tarray(1, A.i64)], lambda xs, to, dfl: A.permute(
        Q.binop(A.mul, A.i64), dfl, A.lam([sh1], lambda ix: A.just(A.sh(A.index(to, A.vexp(ix))))), xs))
    rng = np.random.default_rng(nbins)
    x = rng.integers(0, 1 << 62, N, dtype=np.int64) | 1      # odd factors: the product modulo 2^64 never collapses to 0
    to = rng.integers(0, nbins, N, dtype=np.int64)
    to[rng.random(N) < 0.25] = nbins - 1
    dfl = rng.integers(1, 1000, nbins, dtype=np.int64)
    want = dfl.astype(np.uint64)
    np.multiply.at(want, to, x.astype(np.uint64))
    assert np.array_equal(gpu_ctx.compile(prog)(x, to, dfl).astype(np.uint64), want)


@pytest.mark.gpu
@pytest.mark.parametrize("nbins", [100, 16384, 16385])
def test_float_maximum_through_private_copies(gpu_ctx, nbins):
    x = np.random.default_rng(nbins).normal(size=N).astype(np.float32)
    to = np.random.default_rng(nbins + 1).integers(0, nbins, N, dtype=np.int64)
    dfl = np.full(nbins, -0.5, dtype=np.float32)
    want = dfl.copy()
    np.maximum.at(want, to, x)
    assert np.array_equal(gpu_ctx.compile(_combine_prog(A.max_, A.f32))(x, to, dfl), want)


@pytest.mark.gpu
@pytest.mark.parametrize("order", ["waits", "fences"])
def test_locks_in_memory_under_contention(gpu_ctx, knobs, monkeypatch, order):
    # the private copies switched off: 2^20 sources take turns at the locks of 512 elements (two thousand
    # each), then of 3 -- every update must see the one before it, whichever way the lock is ordered
    if order == "fences":
        monkeypatch.setenv("ACCHIP_LOCK_ORDER", "fences")
    knobs("permute_parts", 0)
    rng = np.random.default_rng(99)
    for n, nbins in ((1 << 20, 512), (1 << 16, 3)):
        x = rng.integers(0, 1 << 30, n, dtype=np.int64)
        to = rng.integers(0, nbins, n, dtype=np.int64)
        a, b = gpu_ctx.compile(_two_smallest(nbins))(x, to)
        m1, m2 = _two_smallest_ref(x, to, nbins, 1 << 40)
        assert np.array_equal(a, m1) and np.array_equal(b, m2), (n, nbins)

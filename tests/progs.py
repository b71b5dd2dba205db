"""Fused terms for the programs the reference's test-suite runs (Test/NoFib/**), written
with the builder the way Trafo.Fusion would hand them to a backend.  Shared by the CPU
tests (oracle vs. golden vectors) and the GPU tests (HIP backend vs. oracle)."""
from __future__ import annotations

from accelerate_amd import ir as A

Int = A.Int


def binop(op, ty):
    return A.lam([ty, ty], lambda x, y: op(ty, x, y))


def fold_op(op, ty, rank, z=None):
    return A.alam([A.tarray(rank, ty)],
                  lambda xs: A.fold(binop(op, ty), None if z is None else A.const(ty, z), xs))


# -- maximum segment sum: fold1 of a non-commutative operator over 4-tuples (Language.hs:491-518)
def mss(ty=Int, rank=1):
    t4 = A.ttup(ty, ty, ty, ty)

    def f(x, y):
        mssx, misx, mcsx, tsx = A.untup(x)
        mssy, misy, mcsy, tsy = A.untup(y)
        mx = lambda a, b: A.max_(ty, a, b)
        return A.tup(mx(mssx, mx(mssy, A.add(ty, mcsx, misy))),
                     mx(misx, A.add(ty, tsx, misy)),
                     mx(mcsy, A.add(ty, mcsx, tsy)),
                     A.add(ty, tsx, tsy))

    def g(x):
        return A.let(ty, A.max_(ty, x, A.const(ty, 0)), lambda y: A.tup(y, y, y, x))

    def first(v):
        return A.untup(v)[0]

    # map fst . fold1 f . map g : the inner map fuses into the fold as a Delayed operand, the
    # outer map is a separate node over the fold's result
    def body(xs):
        sht = A.tshape(rank)
        dl = A.delayed(A.tarray(rank, t4), A.shape(xs),
                       A.lam([sht], lambda ix: A.let(ty, A.index(xs, A.vexp(ix)), g)),
                       A.lam([Int], lambda i: A.let(ty, A.linearindex(xs, i), g)))
        return A.map_(ty, A.lam([t4], first), A.fold(A.lam([t4, t4], f), None, dl))

    return A.alam([A.tarray(rank, ty)], body)


# -- Issue228: fold / fold1 with the non-commutative pair monoid merge
def issue228(seeded):
    t2 = A.ttup(Int, Int)

    def merge(l, r):
        onl, lenl = A.untup(l)
        onr, lenr = A.untup(r)
        return A.tup(A.mul(Int, onl, onr), A.add(Int, A.mul(Int, onl, lenr), lenl))

    z = A.tup(A.constI(1), A.constI(0)) if seeded else None
    return A.alam([A.tarray(1, t2)], lambda xs: A.fold(A.lam([t2, t2], merge), z, xs))


# -- Issue362: scanl1 of component-wise (+) over k-tuples
def tuple_scanl1(k, direction="l"):
    tk = A.ttup(*([Int] * k))

    def f(x, y):
        return A.tup(*[A.add(Int, a, b) for a, b in zip(A.untup(x), A.untup(y))])

    return A.alam([A.tarray(1, tk)], lambda xs: A.scan(direction, A.lam([tk, tk], f), None, xs))


# -- interval monoid of the scan tests (Test/NoFib/Prelude/Scan.hs:745-771): non-commutative
#    iappend (One x y) (One a b) = One x b with Elem = pair; here the "take leftmost first,
#    rightmost second" monoid over pairs, identity-free (used with scan*1 and seeded variants)
def interval_scan(direction, kind, ty=Int, rank=1):
    t2 = A.ttup(ty, ty)

    def f(x, y):
        a, _ = A.untup(x)
        _, d = A.untup(y)
        return A.tup(a, d)

    fn = A.lam([t2, t2], f)
    z = A.tup(A.const(ty, -7), A.const(ty, 9))
    if kind == "scan1":
        return A.alam([A.tarray(rank, t2)], lambda xs: A.scan(direction, fn, None, xs))
    if kind == "scan":
        return A.alam([A.tarray(rank, t2)], lambda xs: A.scan(direction, fn, z, xs))
    return A.alam([A.tarray(rank, t2)], lambda xs: A.scan_(direction, fn, z, xs))


# -- permute const: identity matrix (Language.hs:734-749)
def identity_permute(ty=Int):
    sh1, sh2 = A.tshape(1), A.tshape(2)

    def body(n_arr):
        n = A.index(n_arr, A.nil)
        return A.permute(
            A.lam([ty, A.wild(ty)], lambda x, _: x),
            A.generate(A.tarray(2, ty), A.sh(n, n), A.lam([sh2], lambda ix: A.const(ty, 0))),
            A.lam([sh1], lambda ix: A.just(A.sh(A.untup(ix)[0], A.untup(ix)[0]))),
            A.delayed(A.tarray(1, ty), A.sh(n), A.lam([sh1], lambda ix: A.const(ty, 1)),
                      A.lam([Int], lambda i: A.const(ty, 1))))

    return A.alam([A.tarray(0, Int)], body)


# -- scatter to defaults input = permute const defaults (\ix -> Just (to!ix)) input'
#    with input' = backpermute (shape to `intersect` shape input) id input  (Prelude.hs scatter)
def scatter(ty=Int):
    sh1 = A.tshape(1)

    def body(to, over, xs):
        ext = A.let(sh1, A.shape(to), lambda s1: A.let(sh1, A.shape(xs), lambda s0: A.sh(
            A.min_(Int, A.untup(s1)[0], A.untup(s0)[0]))))
        src = A.delayed(A.tarray(1, ty), ext, A.lam([sh1], lambda ix: A.index(xs, A.vexp(ix))),
                        A.lam([Int], lambda i: A.linearindex(xs, i)))
        return A.permute(A.lam([ty, A.wild(ty)], lambda x, _: A.vexp(x)), over,
                         A.lam([sh1], lambda ix: A.just(A.sh(A.index(to, A.vexp(ix))))), src)

    return A.alam([A.tarray(1, Int), A.tarray(1, ty), A.tarray(1, ty)], body)


# -- accumulate: permute (+) into defaults with an optional drop (Nothing) for negative targets
def accumulate(ty, src_rank, dst_rank):
    shs, shd = A.tshape(src_rank), A.tshape(dst_rank)

    def body(xs, to, defaults):
        def p(ix):
            lin = A.toindex(src_rank, A.shape(xs), A.vexp(ix))
            t = A.linearindex(to, lin)
            return A.let(Int, t, lambda tv: A.cond(
                A.lt(Int, tv, A.constI(0)), A.nothing(shd),
                A.just(A.fromindex(dst_rank, A.shape(defaults), tv))))
        return A.permute(binop(A.add, ty), defaults, A.lam([shs], p), xs)

    return A.alam([A.tarray(src_rank, ty), A.tarray(1, Int), A.tarray(dst_rank, ty)], body)


# -- Issue137: permute with a min-merge combiner over pairs (CAS-free path: per-cell locks)
def issue137():
    t2 = A.ttup(Int, Int)
    sh1 = A.tshape(1)
    inf = A.constI(10000)

    def comb(a12, b12):
        a1, a2 = A.untup(a12)
        b1, b2 = A.untup(b12)
        return A.cond(A.lte(Int, a1, b1), A.tup(a1, A.min_(Int, a2, b1)), A.tup(b1, A.min_(Int, b2, a1)))

    def body(interm, ms):
        src = A.delayed(A.tarray(1, t2), A.shape(interm),
                        A.lam([sh1], lambda ix: A.tup(A.abs_(Int, A.index(interm, A.vexp(ix))), inf)),
                        A.lam([Int], lambda i: A.tup(A.abs_(Int, A.linearindex(interm, i)), inf)))
        return A.permute(A.lam([t2, t2], comb),
                         A.generate(A.tarray(1, t2), A.sh(384), A.lam([sh1], lambda ix: A.tup(inf, inf))),
                         A.lam([sh1], lambda ix: A.just(A.sh(A.index(ms, A.vexp(ix))))), src)

    return A.alam([A.tarray(1, Int), A.tarray(1, Int)], body)


# -- backpermute: transpose (Language.hs:821-842) and gather (Issue185 E)
def transpose(ty=Int):
    sh2 = A.tshape(2)

    def swap(v):
        y, x = A.untup(v)
        return A.sh(x, y)

    return A.alam([A.tarray(2, ty)], lambda m: A.backpermute(
        2, A.let(sh2, A.shape(m), swap), A.lam([sh2], swap), m))


def gather(ty=Int):
    sh1 = A.tshape(1)
    return A.alam([A.tarray(1, Int), A.tarray(1, ty)], lambda frm, xs: A.backpermute(
        1, A.shape(frm), A.lam([sh1], lambda ix: A.sh(A.index(frm, A.vexp(ix)))), xs))


# -- stencils: weighted sum of all taps with distinct weights, any rank / width / boundary
def stencil_weighted(ty, widths, boundary):
    """widths: stencil width per dimension, outermost first (each 3, 5, 7 or 9)."""
    rank = len(widths)

    def pattern(d):
        if d == rank - 1:
            return A.sunit(widths[d], ty)
        return A.stup(*[pattern(d + 1) for _ in range(widths[d])])

    sr = pattern(0)
    counter = [0]

    def weigh(v, d):
        parts = A.untup(v)
        if d == rank - 1:
            terms = []
            for t in parts:
                counter[0] += 1
                terms.append(A.mul(ty, A.const(ty, counter[0]), t))
        else:
            terms = [weigh(p, d + 1) for p in parts]
        acc = terms[0]
        for t in terms[1:]:
            acc = A.add(ty, acc, t)
        return acc

    def f(st):
        counter[0] = 0
        return weigh(st, 0)

    return A.alam([A.tarray(rank, ty)],
                  lambda g: A.stencil(sr, ty, A.lam([A.stencil_type(sr)], f), boundary, g))


def boundary_function(ty, rank):
    """Function boundary: value depends on the (out-of-bounds) index."""
    sht = A.tshape(rank)

    def g(ix):
        acc = A.constI(100)
        for c in A.untup(ix):
            acc = A.add(Int, A.mul(Int, acc, A.constI(3)), c)
        return A.fromintegral(Int, ty, acc)

    return A.function(A.lam([sht], g))


def stencil2_sum(ty, b1, b2):
    sr = A.stup(A.sunit(3, ty), A.sunit(3, ty), A.sunit(3, ty))

    def f(s1, s2):
        a = A.untup(A.untup(s1)[1])  # middle row of the first stencil
        b = A.untup(s2)              # middle column of the second
        top, mid, bot = (A.untup(r)[1] for r in b)
        return A.add(ty, A.add(ty, A.add(ty, a[0], a[2]), A.mul(ty, A.const(ty, 2), mid)), A.sub(ty, top, bot))

    st = A.stencil_type(sr)
    return A.alam([A.tarray(2, ty), A.tarray(2, ty)],
                  lambda x, y: A.stencil2(sr, sr, ty, A.lam([st, st], f), b1, x, b2, y))


# -- whole programs in the shape the reference's nofib "spectral" group has them ------------

def smvm(ty):
    """Spectral/SMVM.hs: foldSeg (+) 0 (zipWith (*) vals (gather inds vec)) segd -- the product
    and the gather are fused into the segmented fold's source; the offsets scan is let-bound."""
    sh1 = A.tshape(1)

    def body(segd, inds, vals, vec):
        def at(ix):
            return A.mul(ty, A.index(vals, A.vexp(ix)), A.index(vec, A.sh(A.index(inds, A.vexp(ix)))))

        def at_lin(i):
            return A.mul(ty, A.linearindex(vals, i), A.index(vec, A.sh(A.linearindex(inds, i))))

        src = A.delayed(A.tarray(1, ty), A.shape(vals), A.lam([sh1], at), A.lam([Int], at_lin))
        return A.alet(A.tarray(1, Int), A.scan("l", binop(A.add, Int), A.constI(0), segd),
                      lambda offs: A.foldseg(Int, binop(A.add, ty), A.const(ty, 0), src, offs))

    return A.alam([A.tarray(1, Int), A.tarray(1, Int), A.tarray(1, ty), A.tarray(1, ty)], body)


def filter_positive(ty=Int):
    """filter (> 0) (Prelude.hs filter): keep-flags, an exclusive scan for the targets and
    the count, a result whose extent is read from the count, a permute that drops the rest."""
    sh1 = A.tshape(1)
    V1, S0 = A.tarray(1, Int), A.tarray(0, Int)

    def body(xs):
        flags = A.map_(Int, A.lam([ty], lambda x: A.cond(A.gt(ty, x, A.const(ty, 0)), A.constI(1), A.constI(0))), xs)

        def with_flags(fl):
            def with_scan(st):
                targets, total = st
                return A.permute(
                    A.lam([ty, A.wild(ty)], lambda x, _: x),
                    A.generate(A.tarray(1, ty), A.sh(A.index(total, A.nil)), A.lam([sh1], lambda ix: A.const(ty, 0))),
                    A.lam([sh1], lambda ix: A.cond(A.eq(Int, A.index(fl, A.vexp(ix)), A.constI(0)), A.nothing(sh1),
                                                   A.just(A.sh(A.index(targets, A.vexp(ix)))))),
                    xs)
            return A.alet(A.tpair(V1, S0), A.scan_("l", binop(A.add, Int), A.constI(0), fl), with_scan)
        return A.alet(V1, flags, with_flags)

    return A.alam([A.tarray(1, ty)], body)


def radix_passes(bits):
    """Spectral/RadixSort.hs, `bits` least-significant-bit passes over Int keys: per pass two
    exclusive scans give the zero-bit keys' and the one-bit keys' places, a permute moves them."""
    sh1 = A.tshape(1)
    V1, S0 = A.tarray(1, Int), A.tarray(0, Int)

    def one_pass(keys, b, rest):
        def bit(k):
            return A.band(Int, A.shr(Int, k, A.constI(b)), A.constI(1))
        ones = A.map_(Int, A.lam([Int], bit), keys)
        zeros = A.map_(Int, A.lam([Int], lambda k: A.sub(Int, A.constI(1), bit(k))), keys)

        def with_zeros(zs):
            zpos, nz = zs

            def with_ones(os_):
                opos, _ = os_

                def dest(ix):
                    k = A.index(keys, A.vexp(ix))
                    return A.just(A.sh(A.cond(A.eq(Int, bit(k), A.constI(0)), A.index(zpos, A.vexp(ix)),
                                              A.add(Int, A.index(nz, A.nil), A.index(opos, A.vexp(ix))))))
                moved = A.permute(A.lam([Int, A.wild(Int)], lambda x, _: x),
                                  A.generate(V1, A.shape(keys), A.lam([sh1], lambda ix: A.constI(0))),
                                  A.lam([sh1], dest), keys)
                return A.alet(V1, moved, rest)
            return A.alet(A.tpair(V1, S0), A.scan_("l", binop(A.add, Int), A.constI(0), ones), with_ones)
        return A.alet(A.tpair(V1, S0), A.scan_("l", binop(A.add, Int), A.constI(0), zeros), with_zeros)

    def build(keys, b):
        if b == bits:
            return keys
        return one_pass(keys, b, lambda moved: build(moved, b + 1))

    return A.alam([V1], lambda keys: build(keys, 0))


# -- segmented scans as Prelude.hs builds them from scan', permute and a flagged scan
#    (mkHeadFlags / mkTailFlags :1364-1389, segmentedL / segmentedR :1395-1407); `ity` is the
#    integral type of the segment descriptor, `rank` the rank of the scanned array
def _seg_flags(seg_src, direction, ity, k):
    """Head flags (left scans) or tail flags (right scans) of a segment descriptor given as an
    operand: permute (+) zeros (\\ix -> Just (offset!ix)) ones.  k receives the array of
    total+1 entries; `init` is left to the consumer (it reads all but the last entry)."""
    sh1 = A.tshape(1)
    V1, S0 = A.tarray(1, ity), A.tarray(0, ity)
    toint = lambda e: e if ity == Int else A.fromintegral(ity, Int, e)

    def with_offsets(st):
        offset, total = st
        ln = lambda: A.index(total, A.nil)

        def target(ix):
            o = A.index(offset, A.vexp(ix))
            return A.just(A.sh(toint(o if direction == "l" else A.sub(ity, A.sub(ity, ln(), A.const(ity, 1)), o))))

        ones = A.delayed(V1, A.shape(offset), A.lam([sh1], lambda ix: A.const(ity, 1)),
                         A.lam([Int], lambda i: A.const(ity, 1)))
        zeros = A.generate(V1, A.sh(A.add(Int, toint(ln()), A.constI(1))), A.lam([sh1], lambda ix: A.const(ity, 0)))
        return A.alet(V1, A.permute(binop(A.add, ity), zeros, A.lam([sh1], target), ones), k)

    return A.alet(A.tpair(V1, S0), A.scan_(direction, binop(A.add, ity), A.const(ity, 0), seg_src), with_offsets)


def _scan1_seg(direction, ty, arr, seg_src, rank=2, ity=Int):
    """scanl1Seg / scanr1Seg (Prelude.hs:1136-1145, 1313-1322) of an array variable:
    map snd . scan1 (segmented f) $ zip (replicate flags) arr, the zip fused into the scan."""
    shr = A.tshape(rank)
    t2 = A.ttup(ity, ty)

    def seg_op(x, y):
        # scanl1: x = running value, y = new element; scanr1: x = new element, y = running value
        (af, av), (bf, bv) = (A.untup(x), A.untup(y)) if direction == "l" else (A.untup(y), A.untup(x))
        f = A.add(ty, av, bv) if direction == "l" else A.add(ty, bv, av)
        return A.tup(A.bor(ity, af, bf), A.cond(A.neq(ity, bf, A.const(ity, 0)), bv, f))

    def with_flags(fl):
        def extent():
            dims = A.untup_shape(arr)
            nfl = A.sub(Int, A.untup_shape(fl)[0], A.constI(1))
            return A.sh(*(dims[:-1] + [A.min_(Int, nfl, dims[-1])]))

        def at(ix):
            x = A.untup(ix)[-1]
            return A.tup(A.index(fl, A.sh(x)), A.index(arr, A.vexp(ix)))

        src = A.delayed(A.tarray(rank, t2), extent(), A.lam([shr], at),
                        A.lam([Int], lambda i: A.let(shr, A.fromindex(rank, extent(), i), at)))
        return A.map_(ty, A.lam([t2], lambda v: A.untup(v)[1]), A.scan(direction, A.lam([t2, t2], seg_op), None, src))

    return _seg_flags(seg_src, direction, ity, with_flags)


def scan1_seg(direction, ty=Int, rank=2, ity=Int):
    return A.alam([A.tarray(rank, ty), A.tarray(1, ity)],
                  lambda arr, seg: _scan1_seg(direction, ty, arr, seg, rank, ity))


def scanl_seg(ty=Int, z=0, rank=2, ity=Int, as_body=False):
    """scanlSeg (Prelude.hs:979-1012): the seed is injected at the head of every segment by a
    permute into an array of seeds, then an inclusive segmented scan over segments one longer."""
    sh1, shr = A.tshape(1), A.tshape(rank)
    V1, M = A.tarray(1, ity), A.tarray(rank, ty)
    toint = lambda e: e if ity == Int else A.fromintegral(ity, Int, e)

    def body(mat, seg):
        def with_flags(fl):
            # (terms are built where they are used: binder levels are fixed at construction)
            nflags = lambda: A.sub(Int, A.untup_shape(fl)[0], A.constI(1))
            outer = lambda: A.untup_shape(mat)[:-1]
            cols = lambda: A.untup_shape(mat)[-1]
            nseg = lambda: A.untup_shape(seg)[0]
            size = lambda: A.shapesize(rank, A.shape(mat))
            taken_sh = lambda: A.sh(*(outer() + [A.min_(Int, nflags(), cols())]))
            filled = lambda: A.generate(M, A.sh(*(outer() + [A.add(Int, cols(), nseg())])),
                                        A.lam([shr], lambda ix: A.const(ty, z)))
            # inc = scanl1 (+) flags, with flags = init fl fused in
            flags = A.delayed(V1, A.sh(nflags()), A.lam([sh1], lambda ix: A.index(fl, A.vexp(ix))),
                              A.lam([Int], lambda i: A.linearindex(fl, i)))

            def with_inc(inc):
                def to(ix):
                    parts = A.untup(ix)
                    x = parts[-1]
                    return A.just(A.sh(*(parts[:-1] + [A.add(Int, x, toint(A.index(inc, A.sh(x))))])))
                # take (length flags) arr
                taken = A.delayed(M, taken_sh(), A.lam([shr], lambda ix: A.index(mat, A.vexp(ix))),
                                  A.lam([Int], lambda i: A.let(shr, A.fromindex(rank, taken_sh(), i),
                                                               lambda ix: A.index(mat, A.vexp(ix)))))
                arr1 = A.permute(A.lam([ty, A.wild(ty)], lambda x, _: x), filled(), A.lam([shr], to), taken)
                seg1 = A.delayed(V1, A.shape(seg),
                                 A.lam([sh1], lambda ix: A.add(ity, A.index(seg, A.vexp(ix)), A.const(ity, 1))),
                                 A.lam([Int], lambda i: A.add(ity, A.linearindex(seg, i), A.const(ity, 1))))
                return A.alet(M, arr1, lambda a1: _scan1_seg("l", ty, a1, seg1, rank, ity))

            empty = A.lor(A.eq(Int, size(), A.constI(0)), A.eq(Int, nflags(), A.constI(0)))
            return A.acond(empty, filled(),
                           A.alet(V1, A.scan("l", binop(A.add, ity), None, flags), with_inc))
        return _seg_flags(seg, "l", ity, with_flags)

    return body if as_body else A.alam([M, V1], body)


# -- SIMD vector element types (Test/NoFib/Prelude/SIMD.hs): extract a component, inject components
def _unpacked(n, ty, v, k):
    """let (c0, .., c{n-1}) = unpack v in k [c0, ..]"""
    return A.let(A.ttup(*[ty] * n), A.vecunpack(n, ty, v), lambda t: k(A.untup(t)))


def _vec_add(n, ty):
    def f(x, y):
        return _unpacked(n, ty, x, lambda xs: _unpacked(n, ty, y, lambda ys: A.vecpack(
            n, ty, A.tup(*[A.add(ty, a, b) for a, b in zip(xs, ys)]))))
    vt = A.tvec(n, ty)
    return A.lam([vt, vt], f)


def vec_extract(n, ty, k, rank=1):
    """map (view _k . unpackVec) xs"""
    vt = A.tvec(n, ty)
    return A.alam([A.tarray(rank, vt)], lambda xs: A.map_(
        ty, A.lam([vt], lambda v: _unpacked(n, ty, v, lambda cs: cs[k])), xs))


def vec_inject(n, ty):
    """zipWith{n} V{n} xs ys ..: one Generate over the intersection after fusion"""
    sh1 = A.tshape(1)
    vt = A.tvec(n, ty)

    def body(*arrs):
        def ext():
            e = A.untup_shape(arrs[0])[0]
            for a in arrs[1:]:
                e = A.min_(Int, e, A.untup_shape(a)[0])
            return A.sh(e)
        return A.generate(A.tarray(1, vt), ext(), A.lam([sh1], lambda ix: A.vecpack(
            n, ty, A.tup(*[A.index(a, A.vexp(ix)) for a in arrs]))))

    return A.alam([A.tarray(1, ty)] * n, body)


def vec_scan(n, ty, direction="l", rank=1):
    """scanl1 / scanr1 of the component-wise sum over Vec n t elements"""
    return A.alam([A.tarray(rank, A.tvec(n, ty))], lambda xs: A.scan(direction, _vec_add(n, ty), None, xs))


def vec_fold(n, ty, rank=2):
    vt = A.tvec(n, ty)
    zero = A.vecpack(n, ty, A.tup(*[A.const(ty, 0)] * n))
    return A.alam([A.tarray(rank, vt)], lambda xs: A.fold(_vec_add(n, ty), zero, xs))


def vec_accumulate(n, ty, nbins):
    """permute (component-wise +) into zeros: no hardware atomic fits, cells are locked"""
    sh1 = A.tshape(1)
    vt = A.tvec(n, ty)
    zero = lambda: A.vecpack(n, ty, A.tup(*[A.const(ty, 0)] * n))
    return A.alam([A.tarray(1, vt), A.tarray(1, Int)], lambda xs, to: A.permute(
        _vec_add(n, ty), A.generate(A.tarray(1, vt), A.sh(nbins), A.lam([sh1], lambda ix: zero())),
        A.lam([sh1], lambda ix: A.just(A.sh(A.index(to, A.vexp(ix))))), xs))


def vec_reverse(n, ty):
    sh1 = A.tshape(1)
    return A.alam([A.tarray(1, A.tvec(n, ty))], lambda xs: A.backpermute(
        1, A.shape(xs), A.lam([sh1], lambda ix: A.sh(A.sub(Int, A.sub(Int, A.untup_shape(xs)[0], A.constI(1)),
                                                            A.untup(ix)[0]))), xs))


def vec_stencil_1d(ty=A.f32):
    """3-point sum of V2 elements, clamp: component-wise left + centre + right"""
    vt = A.tvec(2, ty)

    def f(st):
        l, c, r = A.untup(st)
        return _unpacked(2, ty, l, lambda ls: _unpacked(2, ty, c, lambda cs: _unpacked(2, ty, r, lambda rs: A.vecpack(
            2, ty, A.tup(*[A.add(ty, A.add(ty, ls[k], cs[k]), rs[k]) for k in range(2)])))))

    sr = A.sunit(3, vt)
    return A.alam([A.tarray(1, vt)], lambda xs: A.stencil(sr, vt, A.lam([A.stencil_type(sr)], f), "clamp", xs))


def scanr_seg(ty=Int, z=0, rank=1, ity=Int, as_body=False):
    """scanrSeg (Prelude.hs:1202-1228): as scanlSeg, the seeds injected by a permute whose targets
    are one less than for the left scan, over `drop (sz - length flags) arr`, then scanr1Seg."""
    sh1, shr = A.tshape(1), A.tshape(rank)
    V1, M = A.tarray(1, ity), A.tarray(rank, ty)
    toint = lambda e: e if ity == Int else A.fromintegral(ity, Int, e)

    def body(mat, seg):
        def with_flags(fl):
            nflags = lambda: A.sub(Int, A.untup_shape(fl)[0], A.constI(1))
            outer = lambda: A.untup_shape(mat)[:-1]
            cols = lambda: A.untup_shape(mat)[-1]
            nseg = lambda: A.untup_shape(seg)[0]
            size = lambda: A.shapesize(rank, A.shape(mat))
            dropped = lambda: A.min_(Int, A.sub(Int, cols(), nflags()), cols())     # drop n: n `min` sz
            rest_sh = lambda: A.sh(*(outer() + [A.sub(Int, cols(), dropped())]))
            filled = lambda: A.generate(M, A.sh(*(outer() + [A.add(Int, cols(), nseg())])),
                                        A.lam([shr], lambda ix: A.const(ty, z)))
            flags = A.delayed(V1, A.sh(nflags()), A.lam([sh1], lambda ix: A.index(fl, A.vexp(ix))),
                              A.lam([Int], lambda i: A.linearindex(fl, i)))

            def with_inc(inc):
                def to(ix):
                    parts = A.untup(ix)
                    x = parts[-1]
                    return A.just(A.sh(*(parts[:-1] + [A.sub(Int, A.add(Int, x, toint(A.linearindex(inc, x))), A.constI(1))])))

                def from_rest(ix):
                    parts = A.untup(ix)
                    return A.index(mat, A.sh(*(parts[:-1] + [A.add(Int, parts[-1], dropped())])))
                rest = A.delayed(M, rest_sh(), A.lam([shr], from_rest),
                                 A.lam([Int], lambda i: A.let(shr, A.fromindex(rank, rest_sh(), i), from_rest)))
                arr1 = A.permute(A.lam([ty, A.wild(ty)], lambda x, _: x), filled(), A.lam([shr], to), rest)
                seg1 = A.delayed(V1, A.shape(seg),
                                 A.lam([sh1], lambda ix: A.add(ity, A.index(seg, A.vexp(ix)), A.const(ity, 1))),
                                 A.lam([Int], lambda i: A.add(ity, A.linearindex(seg, i), A.const(ity, 1))))
                return A.alet(M, arr1, lambda a1: _scan1_seg("r", ty, a1, seg1, rank, ity))

            empty = A.lor(A.eq(Int, size(), A.constI(0)), A.eq(Int, nflags(), A.constI(0)))
            return A.acond(empty, filled(),
                           A.alet(V1, A.scan("l", binop(A.add, ity), None, flags), with_inc))
        return _seg_flags(seg, "l", ity, with_flags)

    return body if as_body else A.alam([M, V1], body)


def scan_prime_seg(direction, ty=Int, z=0, rank=2, ity=Int):
    """scanl'Seg / scanr'Seg (Prelude.hs:1041-1094, 1262-1288): the exclusive segmented scan taken
    apart by two backpermutes into the scanned bodies and the per-segment totals."""
    sh1, shr = A.tshape(1), A.tshape(rank)
    V1, S0, M = A.tarray(1, ity), A.tarray(0, ity), A.tarray(rank, ty)
    toint = lambda e: e if ity == Int else A.fromintegral(ity, Int, e)
    inner = scanl_seg(ty, z, rank, ity, True) if direction == "l" else scanr_seg(ty, z, rank, ity, True)
    addi = binop(A.add, ity)

    def body(mat, seg):
        outer = lambda: A.untup_shape(mat)[:-1]
        nseg = lambda: A.untup_shape(seg)[0]
        seg1 = lambda: A.delayed(V1, A.shape(seg),
                                 A.lam([sh1], lambda ix: A.add(ity, A.index(seg, A.vexp(ix)), A.const(ity, 1))),
                                 A.lam([Int], lambda i: A.add(ity, A.linearindex(seg, i), A.const(ity, 1))))

        def with_scanned(arr1):
            def with_starts(st):
                starts, _ = st      # prescanl (+) 0 seg'

                def total_at(ix):
                    parts = A.untup(ix)
                    i = parts[-1]
                    at = A.index(starts, A.sh(i))
                    if direction == "l":    # tails = zipWith (+) seg starts
                        at = A.add(ity, A.index(seg, A.sh(i)), at)
                    return A.sh(*(parts[:-1] + [toint(at)]))
                sums = A.backpermute(rank, A.sh(*(outer() + [nseg()])), A.lam([shr], total_at), arr1)

                def bodies(inc, length):
                    def at(ix):
                        parts = A.untup(ix)
                        i = parts[-1]
                        return A.sh(*(parts[:-1] + [A.add(Int, i, toint(A.index(inc, A.sh(i))))]))
                    return A.apair(A.backpermute(rank, A.sh(*(outer() + [length()])), A.lam([shr], at), arr1), sums)

                if direction == "l":
                    def with_offset(offset):
                        ones = A.delayed(V1, A.shape(seg), A.lam([sh1], lambda ix: A.const(ity, 1)),
                                         A.lam([Int], lambda i: A.const(ity, 1)))
                        marks = A.permute(addi, A.generate(V1, A.sh(A.add(Int, A.shapesize(rank, A.shape(mat)), A.constI(1))),
                                                           A.lam([sh1], lambda ix: A.const(ity, 0))),
                                          A.lam([sh1], lambda ix: A.just(A.sh(toint(A.index(offset, A.vexp(ix)))))), ones)
                        length = lambda: toint(A.index(offset, A.sh(A.sub(Int, A.untup_shape(offset)[0], A.constI(1)))))
                        return A.alet(V1, marks, lambda mk: A.alet(V1, A.scan("l", addi, None, mk),
                                                                   lambda inc: bodies(inc, length)))
                    return A.alet(V1, A.scan("l", addi, None, seg), with_offset)

                def with_flags(fl):
                    nflags = lambda: A.sub(Int, A.untup_shape(fl)[0], A.constI(1))
                    flags = A.delayed(V1, A.sh(nflags()), A.lam([sh1], lambda ix: A.index(fl, A.vexp(ix))),
                                      A.lam([Int], lambda i: A.linearindex(fl, i)))
                    return A.alet(V1, A.scan("l", addi, None, flags), lambda inc: bodies(inc, nflags))
                return _seg_flags(seg, "l", ity, with_flags)
            return A.alet(A.tpair(V1, S0), A.scan_("l", addi, A.const(ity, 0), seg1()), with_starts)

        empty = A.eq(Int, A.shapesize(rank, A.shape(mat)), A.constI(0))
        return A.acond(empty, A.apair(mat, A.generate(M, A.sh(*(outer() + [nseg()])), A.lam([shr], lambda ix: A.const(ty, z)))),
                       A.alet(M, inner(mat, seg), with_scanned))

    return A.alam([M, V1], body)


# -- regression tests of the reference with known answers (Test/NoFib/Issues)
def issue93():
    sh2 = A.tshape(2)
    M = A.tarray(2, Int)
    return A.alam([M], lambda xs: A.permute(
        A.lam([Int, A.wild(Int)], lambda c, _: c),
        A.generate(M, A.shape(xs), A.lam([sh2], lambda ix: A.constI(0))),
        A.lam([sh2], lambda ix: A.just(A.vexp(ix))), xs))


def issue102():
    """p = 3: y = generate (1,3,1) (i == 0 ? 0 : 2) [the reshaped fill 2 inlined], then the
    DFT as fold (+) 0 over coefficients that are all 1 [fill 1 inlined through the replicate],
    reshaped to the shape of y."""
    sh3, sh4 = A.tshape(3), A.tshape(4)
    Y = A.tarray(3, Int)

    def with_y(y):
        def at(ix):
            l, _, r, col = A.untup(ix)
            return A.mul(Int, A.constI(1), A.index(y, A.sh(l, col, r)))
        ext = lambda: A.sh(1, 3, 1, 3)
        src = A.delayed(A.tarray(4, Int), ext(), A.lam([sh4], at),
                        A.lam([Int], lambda i: A.let(sh4, A.fromindex(4, ext(), i), at)))
        return A.reshape(3, A.shape(y), A.reshape(1, A.sh(3), A.fold(binop(A.add, Int), A.constI(0), src)))

    y = A.generate(Y, A.sh(1, 3, 1), A.lam([sh3], lambda ix: A.cond(
        A.eq(Int, A.untup(ix)[1], A.constI(0)), A.constI(0), A.constI(2))))
    return A.alet(Y, y, with_y)


def issue114(kind):
    """Compensated summation over (value, error) pairs: fold1 / scanl1 of a non-commutative add."""
    t2 = A.ttup(A.f32, A.f32)
    f = A.f32

    def add(x, y):
        aval, aerr = A.untup(x)
        bval, berr = A.untup(y)
        return A.let(f, A.add(f, aval, bval), lambda val: A.let(f, A.sub(f, val, aval), lambda det: A.tup(
            val, A.add(f, A.add(f, A.add(f, A.sub(f, aval, A.sub(f, val, det)), A.sub(f, bval, det)), aerr), berr))))
    fn = A.lam([t2, t2], add)
    if kind == "fold1":
        return A.alam([A.tarray(1, t2)], lambda xs: A.fold(fn, None, xs))
    return A.alam([A.tarray(1, t2)], lambda xs: A.scan("l", fn, None, xs))


def issue119_foldall(ty):
    return A.alam([A.tarray(2, ty)], lambda xs: A.fold(
        binop(A.add, ty), A.const(ty, 0), A.reshape(1, A.sh(A.shapesize(2, A.shape(xs))), xs)))


def issue123(n=100):
    sh1 = A.tshape(1)
    ones = A.delayed(A.tarray(1, Int), A.sh(n), A.lam([sh1], lambda ix: A.constI(1)), A.lam([Int], lambda i: A.constI(1)))
    return A.fold(binop(A.add, Int), A.constI(0), ones)


def issue184a(n=1000):
    sh1 = A.tshape(1)

    def f(v):
        def at(ix):
            x = A.untup(ix)[0]
            return A.cond(A.lt(Int, x, A.constI(5)), A.let(Int, A.linearindex(v, x), lambda y: A.mul(Int, y, y)), A.constI(0))
        return A.generate(A.tarray(1, Int), A.sh(n), A.lam([sh1], at))
    return A.alam([A.tarray(1, Int)], f)


def issue287a():
    t6 = A.ttup(*[Int] * 6)

    def f(x, y):
        mi1, l1, c1, r1, li1, ri1 = A.untup(x)
        _, l2, _, r2, _, ri2 = A.untup(y)
        return A.tup(A.max_(Int, mi1, A.add(Int, ri1, l2)), l1, c1, A.mul(Int, r2, r1), li1, ri2)
    return A.alam([A.tarray(1, t6)], lambda xs: A.scan("l", A.lam([t6, t6], f), None, xs))


def issue288():
    t2 = A.ttup(Int, Int)
    loop = lambda e: A.while_(t2, lambda v: A.const(A.u8, 0), lambda v: A.vexp(v), e)
    return A.alam([A.tarray(1, t2)], lambda xs: A.map_(t2, A.lam([t2], lambda v: loop(A.vexp(v))), xs))


def issue364(ty=Int):
    """scanl iappend one: the interval-of-summations monoid with identity `one` and absorbing `top`"""
    t2 = A.ttup(ty, ty)
    c = lambda v: A.const(ty, v)
    is_ = lambda p, v: A.land(A.eq(ty, A.untup(p)[0], c(v)), A.eq(ty, A.untup(p)[1], c(v)))

    def iappend(x, y):
        x1, x2 = A.untup(x)
        y1, y2 = A.untup(y)
        top = A.tup(c(-2), c(-2))
        return A.cond(is_(x, -1), A.vexp(y), A.cond(is_(y, -1), A.vexp(x), A.cond(
            A.lor(is_(x, -2), is_(y, -2)), top,
            A.cond(A.eq(ty, A.add(ty, x2, c(1)), y1), A.tup(x1, y2), top))))
    return A.alam([A.tarray(1, t2)], lambda xs: A.scan("l", A.lam([t2, t2], iappend), A.tup(c(-1), c(-1)), xs))


def issue407(which, ty):
    op = A.isnan if which == "isnan" else A.isinf
    return A.alam([A.tarray(1, ty)], lambda xs: A.map_(A.u8, A.lam([ty], lambda x: op(ty, x)), xs))


def issue409(ty):
    def f(x):
        return A.let(ty, A.recip(ty, x), lambda y: A.let(ty, A.mul(ty, A.neg(ty, y), y), lambda b: A.add(ty, y, A.tanh(ty, b))))
    return A.alam([A.tarray(0, ty)], lambda xs: A.map_(ty, A.lam([ty], f), xs))


def filter_take(n, ty=A.u8):
    """filter (const True) (take n xs) (Issue436): the kept elements and their number"""
    sh1 = A.tshape(1)
    V1, S0 = A.tarray(1, Int), A.tarray(0, Int)

    def body(xs):
        ext = lambda: A.sh(A.min_(Int, A.constI(n), A.untup_shape(xs)[0]))
        flags = A.delayed(V1, ext(), A.lam([sh1], lambda ix: A.constI(1)), A.lam([Int], lambda i: A.constI(1)))
        taken = A.delayed(A.tarray(1, ty), ext(), A.lam([sh1], lambda ix: A.index(xs, A.vexp(ix))),
                          A.lam([Int], lambda i: A.linearindex(xs, i)))

        def with_scan(st):
            targets, total = st
            kept = A.permute(
                A.lam([ty, A.wild(ty)], lambda x, _: x),
                A.generate(A.tarray(1, ty), A.sh(A.index(total, A.nil)), A.lam([sh1], lambda ix: A.const(ty, 0))),
                A.lam([sh1], lambda ix: A.just(A.sh(A.index(targets, A.vexp(ix))))), taken)
            return A.apair(kept, total)
        return A.alet(A.tpair(V1, S0), A.scan_("l", binop(A.add, Int), A.constI(0), flags), with_scan)

    return A.alam([A.tarray(1, ty)], body)


def issue168(which):
    """fill (Z:.1) of a tuple made by iterating a tuple-to-tuple function (Issue168): A applies
    it in the host language, B and C through `iterate` (Prelude.hs: a `while` over (count, value))"""
    F = A.f32
    c = lambda v: A.const(F, v)
    sh1 = A.tshape(1)
    if which == "C":
        ty, seed = A.ttup(*[F] * 6), lambda: A.tup(*[c(v) for v in (6, 5, 4, 3, 2, 1)])
        step = lambda t: A.tup(*reversed(A.untup(t)))
    else:
        ty, seed = A.ttup(F, F), lambda: A.tup(c(2), c(1))
        step = lambda t: A.tup(c(3), A.untup(t)[0])

    def value():
        if which == "A":
            return A.let(ty, seed(), lambda t: step(t))
        st = A.ttup(Int, ty)
        loop = A.while_(st, lambda v: A.lt(Int, A.untup(v)[0], A.constI(1)),
                        lambda v: A.tup(A.add(Int, A.untup(v)[0], A.constI(1)), step(A.untup(v)[1])),
                        A.tup(A.constI(0), seed()))
        return A.let(st, loop, lambda r: A.vexp(A.untup(r)[1]))
    return A.generate(A.tarray(1, ty), A.sh(A.constI(1)), A.lam([sh1], lambda ix: value()))


def issue264_neg(ty):
    """map negate . map negate, fused (Issue264)"""
    return A.alam([A.tarray(1, ty)], lambda xs: A.map_(ty, A.lam([ty], lambda x: A.neg(ty, A.neg(ty, x))), xs))


def issue264_bool(which):
    """not.not over a scalar array of Bool; not (u && v), not (u || v) and their negations
    through zipWith (Issue264)"""
    B = A.u8
    S0 = A.tarray(0, B)
    if which == "not.not":
        return A.alam([S0], lambda xs: A.map_(B, A.lam([B], lambda x: A.lnot(A.lnot(x))), xs))
    op = A.land if "&&" in which else A.lor
    f = (lambda u, v: A.lnot(A.lnot(op(u, v)))) if which.startswith("not(not") else (lambda u, v: A.lnot(op(u, v)))
    return A.alam([S0, S0], lambda xs, ys: A.zipwith(B, A.lam([B, B], f), xs, ys))


def issue286():
    """sum . flatten . map fromIntegral over a matrix of Word8 (Issue286): one fold over a
    delayed, flattened source"""
    sh1 = A.tshape(1)
    get = lambda xs, i: A.fromintegral(A.u8, A.f32, A.linearindex(xs, i))
    return A.alam([A.tarray(2, A.u8)], lambda xs: A.fold(
        binop(A.add, A.f32), A.const(A.f32, 0),
        A.delayed(A.tarray(1, A.f32), A.sh(A.shapesize(2, A.shape(xs))),
                  A.lam([sh1], lambda ix: get(xs, A.untup(ix)[0])), A.lam([Int], lambda i: get(xs, i)))))


def indices_of_truth():
    """map dropBool (afst (filter accept (imap addInds xs))) over a matrix of Bool (Issue427):
    the indexed source is fused into the filter's scans and its permute"""
    B = A.u8
    sh1, sh2 = A.tshape(1), A.tshape(2)
    t3, t2 = A.ttup(Int, Int, B), A.ttup(Int, Int)
    V1, S0, M = A.tarray(1, Int), A.tarray(0, Int), A.tarray(2, Int)

    def body(xs):
        keep = lambda b: A.cond(b, A.constI(1), A.constI(0))
        flags = A.delayed(M, A.shape(xs), A.lam([sh2], lambda ix: keep(A.index(xs, A.vexp(ix)))),
                          A.lam([Int], lambda i: keep(A.linearindex(xs, i))))

        def with_inds_at(ix):
            y, x = A.untup(ix)
            return A.tup(y, x, A.index(xs, A.vexp(ix)))
        with_inds = A.delayed(A.tarray(2, t3), A.shape(xs), A.lam([sh2], with_inds_at),
                              A.lam([Int], lambda i: A.let(sh2, A.fromindex(2, A.shape(xs), i), with_inds_at)))

        def with_rows(st):
            target, length = st

            def with_offsets(so):
                offset, valid = so

                def prj(ix):
                    y, _ = A.untup(ix)
                    return A.cond(A.index(xs, A.vexp(ix)),
                                  A.just(A.sh(A.add(Int, A.linearindex(offset, y), A.index(target, A.vexp(ix))))),
                                  A.nothing(sh1))
                kept = A.permute(A.lam([t3, A.wild(t3)], lambda x, _: A.vexp(x)),
                                 A.generate(A.tarray(1, t3), A.sh(A.index(valid, A.nil)), A.lam([sh1], lambda ix: A.tup(A.undef(Int), A.undef(Int), A.undef(B)))),
                                 A.lam([sh2], prj), with_inds)
                return A.map_(t2, A.lam([t3], lambda v: A.tup(*A.untup(v)[:2])), kept)
            return A.alet(A.tpair(V1, S0), A.scan_("l", binop(A.add, Int), A.constI(0), length), with_offsets)
        return A.alet(A.tpair(M, V1), A.scan_("l", binop(A.add, Int), A.constI(0), flags), with_rows)

    return A.alam([A.tarray(2, B)], body)


def issue437():
    """runN id over (Scalar Float, Matrix Float) (Issue437)"""
    aty = A.tpair(A.tarray(0, A.f32), A.tarray(2, A.f32))
    return A.alam([aty], lambda xs: A.apair(*xs))


def issue517():
    """unit of five `Maybe (Max Float)` combined with (<>) (Issue517): Maybe a is (tag, ((), a)),
    Nothing's payload is undef, and (<>) matches on both tags"""
    F = A.f32
    mb = A.ttup(A.u8, A.ttup(F))
    nothing = lambda: A.tup(A.const(A.u8, 0), A.tup(A.undef(F)))
    just = lambda v: (lambda: A.tup(A.const(A.u8, 1), A.tup(A.const(F, v))))

    def append(a, b):
        def both(x, y):
            both_just = lambda: A.tup(A.const(A.u8, 1), A.tup(A.max_(F, A.untup(A.untup(x)[1])[0], A.untup(A.untup(y)[1])[0])))
            return A.case(A.untup(x)[0], [(0, A.vexp(y)), (1, A.case(A.untup(y)[0], [(0, A.vexp(x)), (1, both_just())]))])
        return A.let(mb, a(), lambda x: A.let(mb, b(), lambda y: both(x, y)))
    t5 = A.ttup(*[mb] * 5)
    return A.unit_(t5, A.tup(append(nothing, nothing), append(nothing, just(2)), append(just(3), nothing),
                             append(just(4), just(5)), append(just(7), just(6))))


def issue551(which):
    """A nine-constructor enumeration (Issue551): word16ToDigit is a chain of conds ending in undef,
    (==) a match on the pair of tags, digitToWord16 a match on the tag"""
    T, W = A.u8, A.u16
    sh1, sh2 = A.tshape(1), A.tshape(2)

    def to_digit(i):
        e = A.undef(T)
        for k in range(8, -1, -1):
            e = A.cond(A.eq(W, i, A.const(W, k)), A.const(T, k), e)
        return e
    to_word = lambda d: A.case(d, [(k, A.const(W, k)) for k in range(9)])
    same = lambda a, b: A.case(a, [(k, A.case(b, [(k, A.const(A.u8, 1))], A.const(A.u8, 0))) for k in range(9)])
    nine = lambda: A.constI(9)
    if which == "eq":
        def at(ix):
            i, j = A.untup(ix)
            return A.let(W, A.fromintegral(Int, W, i), lambda a: A.let(W, A.fromintegral(Int, W, j), lambda b: same(to_digit(a), to_digit(b))))
        return A.generate(A.tarray(2, A.u8), A.sh(nine(), nine()), A.lam([sh2], at))
    digits = A.generate(A.tarray(1, T), A.sh(nine()),
                        A.lam([sh1], lambda ix: A.let(W, A.fromintegral(Int, W, A.untup(ix)[0]), to_digit)))
    return A.alet(A.tarray(1, T), digits, lambda ds: A.map_(W, A.lam([T], to_word), ds))


def issue439():
    S0 = A.tarray(0, A.f32)
    one = A.generate(S0, A.nil, A.lam([A.unit], lambda ix: A.const(A.f32, 1)))
    return A.alet(S0, one, lambda a: A.map_(A.f32, A.lam([A.f32], lambda x: A.mul(A.f32, x, A.const(A.f32, 2))), a))


# -- doctests of Language.hs / Prelude.hs, as the terms fusion would hand over
def fold_all(ty, rank, z):
    """foldAll f z = fold f z . flatten (Prelude.hs:665-672)"""
    return A.alam([A.tarray(rank, ty)], lambda xs: A.fold(
        binop(A.add, ty), A.const(ty, z), xs if rank == 1 else A.reshape(1, A.sh(A.shapesize(rank, A.shape(xs))), xs)))


def all_any(which):
    """all even / any even (Prelude.hs:777-806): and / or over a fused map"""
    sh2 = A.tshape(2)
    B = A.u8
    even = lambda x: A.eq(Int, A.rem(Int, x, A.constI(2)), A.constI(0))
    op, z = (A.land, 1) if which == "all" else (A.lor, 0)

    def body(xs):
        src = A.delayed(A.tarray(2, B), A.shape(xs), A.lam([sh2], lambda ix: even(A.index(xs, A.vexp(ix)))),
                        A.lam([Int], lambda i: even(A.linearindex(xs, i))))
        return A.fold(A.lam([B, B], lambda x, y: op(x, y)), A.const(B, z), src)
    return A.alam([A.tarray(2, Int)], body)


def prescanl_sum():
    """prescanl f e = afst . scanl' f e (Prelude.hs:896-903)"""
    V1, S0 = A.tarray(1, Int), A.tarray(0, Int)
    return A.alam([V1], lambda xs: A.alet(A.tpair(V1, S0), A.scan_("l", binop(A.add, Int), A.constI(0), xs),
                                           lambda st: st[0]))


def postscanl_sum(e):
    """postscanl f e = map (e `f`) . scanl1 f (Prelude.hs:913-921)"""
    return A.alam([A.tarray(1, Int)], lambda xs: A.map_(
        Int, A.lam([Int], lambda x: A.add(Int, A.constI(e), x)), A.scan("l", binop(A.add, Int), None, xs)))


def filter_even():
    """filter even over a vector (Prelude.hs:1623-1662): the kept elements and their number"""
    sh1 = A.tshape(1)
    V1, S0 = A.tarray(1, Int), A.tarray(0, Int)
    even = lambda x: A.eq(Int, A.rem(Int, x, A.constI(2)), A.constI(0))

    def body(xs):
        flags = A.map_(Int, A.lam([Int], lambda x: A.cond(even(x), A.constI(1), A.constI(0))), xs)

        def with_flags(fl):
            def with_scan(st):
                targets, total = st
                kept = A.permute(
                    A.lam([Int, A.wild(Int)], lambda x, _: x),
                    A.generate(V1, A.sh(A.index(total, A.nil)), A.lam([sh1], lambda ix: A.constI(0))),
                    A.lam([sh1], lambda ix: A.cond(A.eq(Int, A.index(fl, A.vexp(ix)), A.constI(0)), A.nothing(sh1),
                                                   A.just(A.sh(A.index(targets, A.vexp(ix)))))), xs)
                return A.apair(kept, total)
            return A.alet(A.tpair(V1, S0), A.scan_("l", binop(A.add, Int), A.constI(0), fl), with_scan)
        return A.alet(V1, flags, with_flags)
    return A.alam([V1], body)


def gather_if(ty=A.f32):
    """gatherIf from mask (> 4) defaults input = zipWith (\\p g -> p ? g) (map pred mask) (zip (gather ..) defaults)"""
    sh1 = A.tshape(1)

    def body(frm, mask, defaults, xs):
        ext = lambda: A.sh(A.min_(Int, A.untup_shape(mask)[0], A.min_(Int, A.untup_shape(frm)[0], A.untup_shape(defaults)[0])))

        def at(ix):
            return A.cond(A.gt(Int, A.index(mask, A.vexp(ix)), A.constI(4)),
                          A.index(xs, A.sh(A.index(frm, A.vexp(ix)))), A.index(defaults, A.vexp(ix)))
        return A.generate(A.tarray(1, ty), ext(), A.lam([sh1], at))
    return A.alam([A.tarray(1, Int), A.tarray(1, Int), A.tarray(1, ty), A.tarray(1, ty)], body)


def scatter_if(ty=Int):
    """scatterIf to mask (> 4) defaults input (Prelude.hs:1788-1793)"""
    sh1 = A.tshape(1)

    def body(to, mask, over, xs):
        ext = A.sh(A.min_(Int, A.untup_shape(to)[0], A.untup_shape(xs)[0]))
        src = A.delayed(A.tarray(1, ty), ext, A.lam([sh1], lambda ix: A.index(xs, A.vexp(ix))),
                        A.lam([Int], lambda i: A.linearindex(xs, i)))
        return A.permute(A.lam([ty, A.wild(ty)], lambda x, _: x), over, A.lam([sh1], lambda ix: A.cond(
            A.gt(Int, A.index(mask, A.vexp(ix)), A.constI(4)), A.just(A.sh(A.index(to, A.vexp(ix)))), A.nothing(sh1))), src)
    return A.alam([A.tarray(1, Int), A.tarray(1, Int), A.tarray(1, ty), A.tarray(1, ty)], body)


def reindex(rank, extent_of, source_of, ty=Int):
    """backpermute with the result's extent and the source index given as functions of lists of
    expressions (outermost first): reverseOn, transposeOn, take, drop, init, tail"""
    shr = A.tshape(rank)
    return A.alam([A.tarray(rank, ty)], lambda xs: A.backpermute(
        rank, A.sh(*extent_of(lambda: A.untup_shape(xs))),
        A.lam([shr], lambda ix: A.sh(*source_of(A.untup(ix), lambda: A.untup_shape(xs)))), xs))


def concat_on(dim):
    """concatOn _1 (the (++) of Prelude.hs:1518-1545) or _2 over matrices: one Generate"""
    sh2 = A.tshape(2)

    def body(m1, m2):
        d1, d2 = (lambda: A.untup_shape(m1)), (lambda: A.untup_shape(m2))
        if dim == 1:    # along the innermost dimension: rows = min, columns = sum
            ext = lambda: A.sh(A.min_(Int, d1()[0], d2()[0]), A.add(Int, d1()[1], d2()[1]))
        else:
            ext = lambda: A.sh(A.add(Int, d1()[0], d2()[0]), A.min_(Int, d1()[1], d2()[1]))

        def at(ix):
            y, x = A.untup(ix)
            if dim == 1:
                return A.cond(A.lt(Int, x, d1()[1]), A.index(m1, A.sh(y, x)), A.index(m2, A.sh(y, A.sub(Int, x, d1()[1]))))
            return A.cond(A.lt(Int, y, d1()[0]), A.index(m1, A.sh(y, x)), A.index(m2, A.sh(A.sub(Int, y, d1()[0]), x)))
        return A.generate(A.tarray(2, Int), ext(), A.lam([sh2], at))
    return A.alam([A.tarray(2, Int), A.tarray(2, Int)], body)


# -- Test/NoFib/Spectral/BlackScholes.hs and Imaginary/{SAXPY,SASUM}.hs
def blackscholes(ty=A.f32):
    t3, t2 = A.ttup(ty, ty, ty), A.ttup(ty, ty)
    c = lambda x: A.const(ty, x)
    mul, add, sub, div = (lambda a, b: A.mul(ty, a, b)), (lambda a, b: A.add(ty, a, b)), \
        (lambda a, b: A.sub(ty, a, b)), (lambda a, b: A.fdiv(ty, a, b))
    let = lambda e, k: A.let(ty, e, k)
    coeff = [0.31938153, -0.356563782, 1.781477937, -1.821255978, 1.330274429]

    def cnd(d, k):
        def tail(kk):
            # horner coeff x = x * foldr1 (\a b -> a + x*b) coeff
            acc = c(coeff[-1])
            for a in coeff[-2::-1]:
                acc = add(c(a), mul(kk, acc))
            poly = mul(kk, acc)
            cn = mul(mul(c(0.39894228040143267793994605993438), A.exp(ty, mul(mul(c(-0.5), d), d))), poly)
            return let(cn, lambda cv: k(A.cond(A.gt(ty, d, c(0)), sub(c(1.0), cv), cv)))
        return let(div(c(1.0), add(c(1.0), mul(c(0.2316419), A.abs_(ty, d)))), tail)

    def go(v):
        price, strike, years = A.untup(v)
        r, vol = c(0.02), c(0.30)
        return let(mul(vol, A.sqrt(ty, years)), lambda vsq: let(
            div(add(A.log(ty, div(price, strike)), mul(add(r, mul(mul(c(0.5), vol), vol)), years)), vsq), lambda d1: let(
                sub(d1, vsq), lambda d2: cnd(d1, lambda c1: let(c1, lambda cd1: cnd(d2, lambda c2: let(c2, lambda cd2: let(
                    mul(strike, A.exp(ty, mul(A.neg(ty, r), years))), lambda xe: A.tup(
                        sub(mul(price, cd1), mul(xe, cd2)),
                        sub(mul(xe, sub(c(1.0), cd2)), mul(price, sub(c(1.0), cd1))))))))))))

    return A.alam([A.tarray(1, t3)], lambda xs: A.map_(t2, A.lam([t3], go), xs))


def saxpy(ty=A.f32):
    """zipWith (\\x y -> alpha * x + y) with alpha a rank-0 argument"""
    return A.alam([A.tarray(0, ty), A.tarray(1, ty), A.tarray(1, ty)], lambda alpha, xs, ys: A.zipwith(
        ty, A.lam([ty, ty], lambda x, y: A.add(ty, A.mul(ty, A.index(alpha, A.nil), x), y)), xs, ys))


def sasum(ty=A.f32):
    """fold (+) 0 . map abs: the map fused into the fold"""
    sh1 = A.tshape(1)

    def body(xs):
        src = A.delayed(A.tarray(1, ty), A.shape(xs), A.lam([sh1], lambda ix: A.abs_(ty, A.index(xs, A.vexp(ix)))),
                        A.lam([Int], lambda i: A.abs_(ty, A.linearindex(xs, i))))
        return A.fold(binop(A.add, ty), A.const(ty, 0), src)
    return A.alam([A.tarray(1, ty)], body)


def accumulate_pairs(t0=A.f32, t1=A.f32, op1=A.add):
    """permute of a component-wise combination over pairs: (a, b) (c, d) -> (a + c, b `op1` d)
    (complex numbers, sum-and-maximum): no cell sees the other component, one atomic each"""
    sh1 = A.tshape(1)
    t2 = A.ttup(t0, t1)

    def f(x, y):
        a, b = A.untup(x)
        c, d = A.untup(y)
        return A.tup(A.add(t0, a, c), op1(t1, d, b))
    return A.alam([A.tarray(1, t2), A.tarray(1, Int), A.tarray(1, t2)], lambda xs, to, dfl: A.permute(
        A.lam([t2, t2], f), dfl, A.lam([sh1], lambda ix: A.just(A.sh(A.index(to, A.vexp(ix))))), xs))


def replicate_(spec, slix, src_rank, out_rank, ty=Int):
    """Replicate as fusion leaves it (Trafo/Fusion.hs replicateD): a Backpermute whose extent is
    IndexFull of the source's shape and whose index map is IndexSlice.  spec lists all / fixed
    from the innermost dimension outwards, slix is the matching slice index."""
    sho = A.tshape(out_rank)
    return A.alam([A.tarray(src_rank, ty)], lambda xs: A.backpermute(
        out_rank, A.indexfull(spec, slix(), A.shape(xs)),
        A.lam([sho], lambda ix: A.indexslice(spec, slix(), A.vexp(ix))), xs))


def slice_of(spec, slix, src_rank, out_rank, ty=Int):
    """Slice as fusion leaves it (sliceD): extent IndexSlice of the source's shape, index map IndexFull"""
    sho = A.tshape(out_rank)
    return A.alam([A.tarray(src_rank, ty)], lambda xs: A.backpermute(
        out_rank, A.indexslice(spec, slix(), A.shape(xs)),
        A.lam([sho], lambda ix: A.indexfull(spec, slix(), A.vexp(ix))), xs))


def filter_rows(pred, ty=Int):
    """filter over a matrix (compact, Prelude.hs:1670-1686): per-row exclusive scans of the keep
    flags give the targets inside a row and the row's count, an exclusive scan of the counts
    the rows' offsets, a permute gathers the kept elements; returns (elements, counts per row)."""
    sh1, sh2 = A.tshape(1), A.tshape(2)
    V1, S0, M = A.tarray(1, Int), A.tarray(0, Int), A.tarray(2, Int)

    def body(xs):
        flags = A.delayed(M, A.shape(xs),
                          A.lam([sh2], lambda ix: A.cond(pred(A.index(xs, A.vexp(ix))), A.constI(1), A.constI(0))),
                          A.lam([Int], lambda i: A.cond(pred(A.linearindex(xs, i)), A.constI(1), A.constI(0))))

        def with_rows(st):
            target, length = st

            def with_offsets(so):
                offset, valid = so

                def prj(ix):
                    y, _ = A.untup(ix)
                    return A.cond(pred(A.index(xs, A.vexp(ix))),
                                  A.just(A.sh(A.add(Int, A.linearindex(offset, y), A.index(target, A.vexp(ix))))),
                                  A.nothing(sh1))
                result = A.permute(A.lam([ty, A.wild(ty)], lambda x, _: x),
                                   A.generate(A.tarray(1, ty), A.sh(A.index(valid, A.nil)), A.lam([sh1], lambda ix: A.undef(ty))),
                                   A.lam([sh2], prj), xs)
                return A.apair(result, length)
            return A.alet(A.tpair(V1, S0), A.scan_("l", binop(A.add, Int), A.constI(0), length), with_offsets)
        return A.alet(A.tpair(M, V1), A.scan_("l", binop(A.add, Int), A.constI(0), flags), with_rows)

    return A.alam([A.tarray(2, ty)], body)


def indexed(rank, ty=A.f32):
    """indexed = imap (\\ix x -> (ix, x)) (Prelude.hs:157-177): a Transform over the source"""
    shr = A.tshape(rank)
    out = A.ttup(shr, ty)
    return A.alam([A.tarray(rank, ty)], lambda xs: A.generate(
        A.tarray(rank, out), A.shape(xs), A.lam([shr], lambda ix: A.tup(A.vexp(ix), A.index(xs, A.vexp(ix))))))


def enum_from_step_n(rank, dims, ty, x0, dx):
    """enumFromStepN sh x y = reshape sh (generate (size sh) (\\i -> x + fromIntegral i * y))  (Prelude.hs:1475-1488)"""
    sh1 = A.tshape(1)
    n = 1
    for d in dims:
        n *= d
    conv = (lambda i: A.fromintegral(Int, ty, i)) if ty in A.INTEGRAL else (lambda i: A.tofloating(Int, ty, i))
    gen = A.generate(A.tarray(1, ty), A.sh(n), A.lam([sh1], lambda ix: A.add(
        ty, A.const(ty, x0), A.mul(ty, conv(A.untup(ix)[0]), A.const(ty, dx)))))
    return A.reshape(rank, A.sh(*dims), gen)


def misc_cache(which):
    """Test/NoFib/Misc/Cache.hs: two nodes with the same scalar code but different extent
    expressions; a kernel cache whose key leaves the extents out must still give each its own."""
    sh1 = A.tshape(1)
    V, S0 = A.tarray(1, A.f32), A.tarray(0, A.f32)
    plus = binop(A.add, A.f32)

    def body(a, b):
        n, m = (lambda: A.untup_shape(a)[0]), (lambda: A.untup_shape(b)[0])
        if which == "generate":
            f = lambda: A.lam([sh1], lambda ix: A.index(a, A.sh(A.rem(Int, A.untup(ix)[0], A.constI(10)))))
            c = A.generate(V, A.sh(A.add(Int, n(), m())), f())
            d = lambda: A.generate(V, A.sh(A.mul(Int, A.constI(3), n())), f())
        else:
            ident = lambda: A.lam([sh1], lambda ix: A.vexp(ix))
            c = A.backpermute(1, A.sh(A.min_(Int, n(), m())), ident(), a)
            d = lambda: A.backpermute(1, A.sh(n()), ident(), a)
        return A.alet(V, c, lambda cv: A.alet(V, d(), lambda dv: A.zipwith(
            A.f32, plus, A.fold(plus, A.const(A.f32, 0), cv), A.fold(plus, A.const(A.f32, 0), dv))))
    return A.alam([V, V], body)


def long_array_programs(big, n):
    """Three closed programs over arrays made on the device: fold (+) 7 over the delayed source
    i -> i .&. 255 of `big` elements; the last 8 elements of map (+1) over `big` manifest bytes
    i .&. 255; the last 6 elements of scanl1 (+) over n Int32 ones."""
    sh1 = A.tshape(1)
    low = lambda i: A.band(Int, i, A.constI(255))
    src = A.delayed(A.tarray(1, Int), A.sh(A.constI(big)), A.lam([sh1], lambda ix: low(A.untup(ix)[0])), A.lam([Int], low))
    fold = A.fold(binop(A.add, Int), A.constI(7), src)
    B, I32 = A.u8, A.i32
    tail = lambda ys, m, k: A.backpermute(1, A.sh(A.constI(k)), A.lam(
        [sh1], lambda ix: A.sh(A.add(Int, A.untup(ix)[0], A.constI(m - k)))), ys)
    bytes_ = A.generate(A.tarray(1, B), A.sh(A.constI(big)), A.lam([sh1], lambda ix: A.fromintegral(Int, B, low(A.untup(ix)[0]))))
    far_end = A.alet(A.tarray(1, B), bytes_, lambda xs: A.alet(
        A.tarray(1, B), A.map_(B, A.lam([B], lambda x: A.add(B, x, A.const(B, 1))), xs), lambda ys: tail(ys, big, 8)))
    ones = A.generate(A.tarray(1, I32), A.sh(A.constI(n)), A.lam([sh1], lambda ix: A.const(I32, 1)))
    scan_end = A.alet(A.tarray(1, I32), ones, lambda xs: A.alet(
        A.tarray(1, I32), A.scan("l", binop(A.add, I32), None, xs), lambda ys: tail(ys, n, 6)))
    return fold, far_end, scan_end


def long_fold_expected(big):
    return 7 + (big // 256) * (255 * 128) + sum(range(big % 256))


# -- fold1Seg (Test/NoFib/Prelude/Fold.hs:102-121): the surface function scans the lengths into
#    offsets first (Prelude.hs:730-737), the node consumes offsets and has no seed
def fold1seg_sum(ty=Int, rank=1, ity=Int):
    return A.alam([A.tarray(rank, ty), A.tarray(1, ity)], lambda vals, seg: A.alet(
        A.tarray(1, ity), A.scan("l", binop(A.add, ity), A.const(ity, 0), seg),
        lambda offs: A.foldseg(ity, binop(A.add, ty), None, vals, offs)))


def fold1seg_interval(rank=1, ty=Int, ity=Int):
    """fold1Seg of the interval monoid over pairs: (a, _) <> (_, d) = (a, d); neither commutative
    nor indifferent to where a segment starts and ends"""
    t2 = A.ttup(ty, ty)

    def f(x, y):
        a, _ = A.untup(x)
        _, d = A.untup(y)
        return A.tup(a, d)

    return A.alam([A.tarray(rank, t2), A.tarray(1, ity)], lambda vals, seg: A.alet(
        A.tarray(1, ity), A.scan("l", binop(A.add, ity), A.const(ity, 0), seg),
        lambda offs: A.foldseg(ity, A.lam([t2, t2], f), None, vals, offs)))


# -- Transform (AST.hs:289-296): out[ix] = f (a ! p ix); here the transpose of 3 * x + 1
def transform_transpose_affine(ty=Int):
    sh2 = A.tshape(2)

    def swap(v):
        y, x = A.untup(v)
        return A.sh(x, y)

    return A.alam([A.tarray(2, ty)], lambda m: A.transform(
        A.tarray(2, ty), A.let(sh2, A.shape(m), swap), A.lam([sh2], swap),
        A.lam([ty], lambda x: A.add(ty, A.mul(ty, A.const(ty, 3), x), A.const(ty, 1))), m))


def transform_gather_scale(ty=A.f32):
    """Transform with a data-dependent index function: out[i] = 0.5 * xs[from[i]]"""
    sh1 = A.tshape(1)
    return A.alam([A.tarray(1, Int), A.tarray(1, ty)], lambda frm, xs: A.transform(
        A.tarray(1, ty), A.shape(frm), A.lam([sh1], lambda ix: A.sh(A.index(frm, A.vexp(ix)))),
        A.lam([ty], lambda x: A.mul(ty, A.const(ty, 0.5), x)), xs))


# -- a scan whose combination function looks its result up in a table indexed by both operands
#    (composition of finite-state transitions): the function must only ever be applied to values
#    of the array, or the lookup leaves the table
def table_scan(k, direction="l", kind="scan1"):
    sh1 = A.tshape(1)

    def body(tbl, xs):
        f = A.lam([Int, Int], lambda a, b: A.index(tbl, A.sh(A.add(Int, A.mul(Int, a, A.constI(k)), b))))
        if kind == "scan1":
            return A.scan(direction, f, None, xs)
        return A.scan(direction, f, A.constI(0), xs)

    return A.alam([A.tarray(1, Int), A.tarray(1, Int)], body)

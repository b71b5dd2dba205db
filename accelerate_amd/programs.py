"""The fused terms the reference's optimiser produces for common surface programs.

Each function returns the textual DelayedOpenAfun that `Trafo.convertAfun` hands to a
backend for the named surface program (shapes of the terms derived from
Trafo/Fusion.hs:139-216, 1195-1233 and Prelude.hs); they are what the benchmark and the
parity tests feed to both this backend and the oracle.
"""
from __future__ import annotations

from . import ir as A


def _binop(op, ty):
    return A.lam([ty, ty], lambda x, y: op(ty, x, y))


def dotp(ty=A.f32):
    """fold (+) 0 (zipWith (*) xs ys)  (README.md:53-54): the multiply is fused into the
    reduction as a Delayed operand; xs is a1, ys is a0."""
    return A.alam([A.tarray(1, ty), A.tarray(1, ty)], lambda xs, ys: A.fold(
        _binop(A.add, ty), A.const(ty, 0),
        A.delayed_zipwith(ty, 1, lambda x, y: A.mul(ty, x, y), xs, ty, ys, ty)))


def fold_sum(ty, rank, z=0):
    """fold (+) z over the innermost dimension of a manifest array."""
    return A.alam([A.tarray(rank, ty)], lambda xs: A.fold(_binop(A.add, ty), A.const(ty, z), xs))


def fold1_op(op, ty, rank):
    return A.alam([A.tarray(rank, ty)], lambda xs: A.fold(_binop(op, ty), None, xs))


def scanl1_sum(ty, rank=1):
    """scanl1 (+): Scan LeftToRight (+) Nothing (Manifest (Avar a0))."""
    return A.alam([A.tarray(rank, ty)], lambda xs: A.scan("l", _binop(A.add, ty), None, xs))


def scan_sum(direction, ty, rank=1, z=0):
    return A.alam([A.tarray(rank, ty)], lambda xs: A.scan(direction, _binop(A.add, ty), A.const(ty, z), xs))


def scan1_sum(direction, ty, rank=1):
    return A.alam([A.tarray(rank, ty)], lambda xs: A.scan(direction, _binop(A.add, ty), None, xs))


def scan_prime_sum(direction, ty, rank=1, z=0):
    return A.alam([A.tarray(rank, ty)], lambda xs: A.scan_(direction, _binop(A.add, ty), A.const(ty, z), xs))


def foldseg_sum(ty=A.i32, ity=A.i32, rank=1, z=0):
    """foldSeg (+) z vals seg = foldSeg' (+) z vals (scanl (+) 0 seg)  (Prelude.hs:710-717):
    the offsets scan is a separate let-bound node, the segmented fold consumes offsets."""
    return A.alam([A.tarray(rank, ty), A.tarray(1, ity)], lambda vals, seg: A.alet(
        A.tarray(1, ity), A.scan("l", _binop(A.add, ity), A.const(ity, 0), seg),
        lambda offs: A.foldseg(ity, _binop(A.add, ty), A.const(ty, z), vals, offs)))


def histogram(nbins, key_ty=A.i32, ty=A.i32):
    """permute (+) (fill (I1 nbins) 0) (\\ix -> Just (I1 (fromIntegral (keys!ix)))) ones
    (Language.hs:716-728): defaults are a Generate node, the ones are a fused constant."""
    sh1 = A.tshape(1)
    return A.alam([A.tarray(1, key_ty)], lambda keys: A.permute(
        _binop(A.add, ty),
        A.generate(A.tarray(1, ty), A.sh(nbins), A.lam([sh1], lambda ix: A.const(ty, 0))),
        A.lam([sh1], lambda ix: A.just(A.tup(A.fromintegral(key_ty, A.Int, A.index(keys, A.vexp(ix)))))),
        A.delayed(A.tarray(1, ty), A.shape(keys), A.lam([sh1], lambda ix: A.const(ty, 1)),
                  A.lam([A.Int], lambda i: A.const(ty, 1)))))


def jacobi_step(ty=A.f32):
    """stencil (\\((_,t,_),(l,_,r),(_,b,_)) -> 0.25 * (t + l + r + b)) clamp: the constant is
    moved to the left of (*) by the simplifier (Trafo/Algebra.hs:157-192) and the user's
    association of the sum is kept."""
    sr = A.stup(A.sunit(3, ty), A.sunit(3, ty), A.sunit(3, ty))

    def f(st):
        (r0, r1, r2) = A.untup(st)
        _, t, _ = A.untup(r0)
        l, _, r = A.untup(r1)
        _, b, _ = A.untup(r2)
        return A.mul(ty, A.const(ty, 0.25), A.add(ty, A.add(ty, A.add(ty, t, l), r), b))

    return A.alam([A.tarray(2, ty)], lambda g: A.stencil(sr, ty, A.lam([A.stencil_type(sr)], f), A.clamp, g))


def map_affine(ty=A.f32):
    """map (\\x -> 2*x + 1): one read and one write per element."""
    return A.alam([A.tarray(1, ty)], lambda xs: A.map_(
        ty, A.lam([ty], lambda x: A.add(ty, A.mul(ty, A.const(ty, 2), x), A.const(ty, 1))), xs))
